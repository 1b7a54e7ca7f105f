// Device-side helpers for gfx950 (CDNA4, wave64): cross-lane reductions through DPP /
// ds_swizzle, segmented scans, small utilities.  The reference's counterparts are the
// __shfl_xor loops in include/alphasparse/common.h:457-605; nothing here is shared with them.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace asx {

constexpr int kWave = 64;

// ---- DPP moves -------------------------------------------------------------------------
// dpp_ctrl encodings: quad_perm = 0x00..0xFF, row_shr:n = 0x110+n, row_mirror = 0x140,
// row_half_mirror = 0x141, row_bcast15 = 0x142, row_bcast31 = 0x143.
template <int CTRL>
__device__ __forceinline__ int dpp_i32(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xF, 0xF, true);
}
template <int CTRL>
__device__ __forceinline__ float dpp(float v)
{
    return __int_as_float(dpp_i32<CTRL>(__float_as_int(v)));
}
template <int CTRL>
__device__ __forceinline__ double dpp(double v)
{
    int lo = dpp_i32<CTRL>(__double2loint(v));
    int hi = dpp_i32<CTRL>(__double2hiint(v));
    return __hiloint2double(hi, lo);
}

// ds_swizzle, bit-mask mode: lane' = ((lane & and) | or) ^ xor inside groups of 32
template <int PATTERN>
__device__ __forceinline__ float swz(float v)
{
    return __int_as_float(__builtin_amdgcn_ds_swizzle(__float_as_int(v), PATTERN));
}
template <int PATTERN>
__device__ __forceinline__ double swz(double v)
{
    int lo = __builtin_amdgcn_ds_swizzle(__double2loint(v), PATTERN);
    int hi = __builtin_amdgcn_ds_swizzle(__double2hiint(v), PATTERN);
    return __hiloint2double(hi, lo);
}

// Sum over aligned groups of W consecutive lanes (W = 1,2,4,...,64); every lane of a
// group ends up holding the group's sum.  Fixed pairing order, so results are reproducible.
template <int W, typename T>
__device__ __forceinline__ T group_sum(T v)
{
    if (W >= 2) v += dpp<0xB1>(v);   // quad_perm [1,0,3,2] : lane ^ 1
    if (W >= 4) v += dpp<0x4E>(v);   // quad_perm [2,3,0,1] : lane ^ 2
    if (W >= 8) v += dpp<0x141>(v);  // row_half_mirror     : other quad of the 8
    if (W >= 16) v += dpp<0x140>(v); // row_mirror          : other half of the 16
    if (W >= 32) v += swz<0x401F>(v); // xor 16 inside 32
    if (W >= 64) v += __shfl_xor(v, 32, 64);
    return v;
}

// ---- segmented inclusive scan over a wave -------------------------------------------------
// Keys are non-decreasing across lanes.  After the call `v` holds the sum of the values of
// the run of equal keys that ends at this lane (restricted to the wave).
template <typename T>
__device__ __forceinline__ T wave_segscan_incl(int key, T v)
{
    const int lane = __lane_id();
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        int k2 = __shfl_up(key, d, kWave);
        T v2 = __shfl_up(v, d, kWave);
        if (lane >= d && k2 == key) v += v2;
    }
    return v;
}

// ---- segmented inclusive sum over a wave, DPP only (no LDS traffic) ---------------------------
// Lanes whose `closed` is set start a new segment (their v already is the sum from the segment's
// start inside the lane); lane 0 must be closed.  Returns, per lane, the sum of v from the nearest
// closed lane at or below it up to itself.  Hillis-Steele over rows of 16 lanes (row_shr), then
// row_bcast15 / row_bcast31 across rows; stops as soon as every lane has a segment start in reach
// (after one step when nearly every lane is closed).  Lanes a move does not reach receive 0.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ int dpp0_i32(int v)
{
    return __builtin_amdgcn_update_dpp(0, v, CTRL, ROW_MASK, 0xF, false);
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp0(float v)
{
    return __int_as_float(dpp0_i32<CTRL, ROW_MASK>(__float_as_int(v)));
}
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ double dpp0(double v)
{
    const int lo = dpp0_i32<CTRL, ROW_MASK>(__double2loint(v));
    const int hi = dpp0_i32<CTRL, ROW_MASK>(__double2hiint(v));
    return __hiloint2double(hi, lo);
}
template <typename T>
__device__ __forceinline__ T wave_segsum_dpp(T v, bool closed)
{
    int f = closed ? 1 : 0;
#define ASX_SEG_STEP(CTRL, ROW_MASK)                        \
    {                                                       \
        if (__ballot(f == 0) == 0) return v;                \
        const T v2 = dpp0<CTRL, ROW_MASK>(v);               \
        const int f2 = dpp0_i32<CTRL, ROW_MASK>(f);         \
        v = f ? v : v + v2;                                 \
        f |= f2;                                            \
    }
    ASX_SEG_STEP(0x111, 0xF)  // row_shr:1
    ASX_SEG_STEP(0x112, 0xF)  // row_shr:2
    ASX_SEG_STEP(0x114, 0xF)  // row_shr:4
    ASX_SEG_STEP(0x118, 0xF)  // row_shr:8
    ASX_SEG_STEP(0x142, 0xA)  // row_bcast15 into rows 1 and 3
    ASX_SEG_STEP(0x143, 0xC)  // row_bcast31 into rows 2 and 3
#undef ASX_SEG_STEP
    return v;
}
// value of the lane below (lane 0 receives 0): wave_shr:1
template <typename T>
__device__ __forceinline__ T wave_shift_up1(T v)
{
    return dpp0<0x138, 0xF>(v);
}

// value of one lane (a constant), in every lane
template <typename T>
__device__ __forceinline__ T wave_readlane(T v, int lane);
template <>
__device__ __forceinline__ float wave_readlane<float>(float v, int lane)
{
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), lane));
}
template <>
__device__ __forceinline__ double wave_readlane<double>(double v, int lane)
{
    const int lo = __builtin_amdgcn_readlane(__double2loint(v), lane);
    const int hi = __builtin_amdgcn_readlane(__double2hiint(v), lane);
    return __hiloint2double(hi, lo);
}

template <typename T>
__device__ __forceinline__ T fma_t(T a, T b, T c);
template <>
__device__ __forceinline__ float fma_t<float>(float a, float b, float c)
{
    return __builtin_fmaf(a, b, c);
}
template <>
__device__ __forceinline__ double fma_t<double>(double a, double b, double c)
{
    return __builtin_fma(a, b, c);
}

__host__ __device__ __forceinline__ int64_t ceil_div64(int64_t a, int64_t b) { return (a + b - 1) / b; }

}  // namespace asx
