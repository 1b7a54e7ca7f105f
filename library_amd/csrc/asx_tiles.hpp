// Device code shared by the kernels that stream a matrix as tiles of 256 stored elements with a
// 16-bit local column and a "first element of a run" flag per element, gather x from LDS and sum
// runs (asx_sliced.hip: runs = (row, slice) pairs; asx_window.hip: runs = rows).
#pragma once
#include "asx_internal.hpp"

namespace asx {

// Position of logical element e (= 4*lane + j) of a tile in the tile's value storage: the order
// in which 16-byte loads at consecutive lanes deliver 4 consecutive elements to each lane.
template <typename T>
__host__ __device__ __forceinline__ int tile_val_pos(int e)
{
    if (sizeof(T) == 8) {  // two loads of 2 doubles: [half][lane][2]
        const int lane = e >> 2, j = e & 3;
        return (j >> 1) * 128 + lane * 2 + (j & 1);
    }
    return e;  // one load of 4 floats
}

// Where the column | flag word of the tile's p-th slot (in the order of A's stored elements) lies
// in a tile whose lanes hold two pairs of consecutive slots, 2 lane .. 2 lane + 1 and
// 128 + 2 lane .. 128 + 2 lane + 1 (tile_reduce_halves): the lane's four words are consecutive.
__host__ __device__ __forceinline__ int tile_halves_pos(int p)
{
    return ((p & 127) >> 1) * 4 + (p >> 7) * 2 + (p & 1);
}

template <typename T>
struct TileValues;
template <>
struct TileValues<double> {
    static __device__ __forceinline__ void load(const double *tile, int lane, double v[4])
    {
        typedef double f64x2 __attribute__((ext_vector_type(2)));
        const f64x2 *q = reinterpret_cast<const f64x2 *>(tile);
        const f64x2 a = __builtin_nontemporal_load(q + lane);
        const f64x2 b = __builtin_nontemporal_load(q + 64 + lane);
        v[0] = a.x, v[1] = a.y, v[2] = b.x, v[3] = b.y;
    }
};
template <>
struct TileValues<float> {
    static __device__ __forceinline__ void load(const float *tile, int lane, float v[4])
    {
        typedef float f32x4 __attribute__((ext_vector_type(4)));
        const f32x4 a = __builtin_nontemporal_load(reinterpret_cast<const f32x4 *>(tile) + lane);
        v[0] = a.x, v[1] = a.y, v[2] = a.z, v[3] = a.w;
    }
};

__device__ __forceinline__ int lanes_below(unsigned long long mask)
{
    return __builtin_amdgcn_mbcnt_hi((unsigned)(mask >> 32), __builtin_amdgcn_mbcnt_lo((unsigned)mask, 0));
}

// One tile's stored elements as the loads deliver them.
template <typename T>
struct Tile {
    uint32_t c01, c23;  // 4 x (local column | run start << 15)
    T v[4];
    int32_t base;  // per-tile word: index of the tile's first partial sum (sliced), first row (window)
};
template <typename T>
__device__ __forceinline__ void tile_load(Tile<T> &tl, int32_t t, int lane, const uint16_t *__restrict__ cf,
                                          const T *__restrict__ val, const int32_t *__restrict__ tile_word)
{
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    const u32x2 cw = __builtin_nontemporal_load(reinterpret_cast<const u32x2 *>(cf + (int64_t)t * kSlicedTile) + lane);
    tl.c01 = cw.x;
    tl.c23 = cw.y;
    TileValues<T>::load(val + (int64_t)t * kSlicedTile, lane, tl.v);
    tl.base = tile_word[t];
}

// Products, running sums and wave scan of one tile; `emit(wanted, rank, sum)` is called five times
// by every lane, `wanted` on the lanes that close a run: rank = position of the run in the tile (a
// tile starts with a run start; meaningless where not wanted).  Whether an emitter branches on
// `wanted` or stores to a spare place instead is its own choice: a branch that depends on the lane
// makes the compiler restructure the loops around it, and with them what it knows about which
// loads are still in flight.  Returns the number of runs.  Lane l holds elements 4l .. 4l+3; a run
// start closes the run before it; lane 63 closes the last one.
template <typename T, typename Emit>
__device__ __forceinline__ int tile_reduce(const Tile<T> &tl, int lane, const T *xs, Emit emit)
{
    const bool f0 = (tl.c01 >> 15) & 1, f1 = tl.c01 >> 31, f2 = (tl.c23 >> 15) & 1, f3 = tl.c23 >> 31;
    const T p0 = tl.v[0] * xs[tl.c01 & 0x7fff], p1 = tl.v[1] * xs[(tl.c01 >> 16) & 0x7fff];
    const T p2 = tl.v[2] * xs[tl.c23 & 0x7fff], p3 = tl.v[3] * xs[(tl.c23 >> 16) & 0x7fff];
    // running sums that restart at every run start
    const T r0 = p0;
    const T r1 = f1 ? p1 : r0 + p1;
    const T r2 = f2 ? p2 : r1 + p2;
    const T r3 = f3 ? p3 : r2 + p3;
    const int nh = (int)f0 + (int)f1 + (int)f2 + (int)f3;
    const unsigned long long m0 = __ballot(f0), m1 = __ballot(f1), m2 = __ballot(f2), m3 = __ballot(f3);
    const int before = lanes_below(m0) + lanes_below(m1) + lanes_below(m2) + lanes_below(m3);
    const int total = __popcll(m0) + __popcll(m1) + __popcll(m2) + __popcll(m3);
    // sum of the run that is open at the end of each lane, over the lanes it spans
    const T open = wave_segsum_dpp<T>(r3, nh != 0);
    const T cin = wave_shift_up1<T>(open);  // what earlier lanes hold of the run open at this lane's start
    int hb = before;
    emit(f0 && hb > 0, hb - 1, cin);
    hb += f0;
    emit(f1, hb - 1, f0 ? r0 : cin + r0);
    hb += f1;
    emit(f2, hb - 1, (f0 | f1) ? r1 : cin + r1);
    hb += f2;
    emit(f3, hb - 1, (f0 | f1 | f2) ? r2 : cin + r2);
    emit(lane == kWave - 1, total - 1, open);
    return total;
}

// tile_reduce for a tile whose lane l holds slots 2l, 2l + 1 (c01, v[0..1]) and 128 + 2l,
// 128 + 2l + 1 (c23, v[2..3]): two 16-byte loads per lane that each read 1 KiB of consecutive
// values, where four consecutive doubles a lane would take two loads that each skip every other
// 16 bytes.  The halves are summed side by side (two scans over the wave, independent of one
// another); the run that the first half leaves open goes on through the lanes of the second half
// below its first run start.  Same calls of `emit`, same return value.
template <typename T, typename Emit>
__device__ __forceinline__ int tile_reduce_halves(const Tile<T> &tl, int lane, const T *xs, Emit emit)
{
    const bool f0 = (tl.c01 >> 15) & 1, f1 = tl.c01 >> 31, f2 = (tl.c23 >> 15) & 1, f3 = tl.c23 >> 31;
    const T p0 = tl.v[0] * xs[tl.c01 & 0x7fff], p1 = tl.v[1] * xs[(tl.c01 >> 16) & 0x7fff];
    const T p2 = tl.v[2] * xs[tl.c23 & 0x7fff], p3 = tl.v[3] * xs[(tl.c23 >> 16) & 0x7fff];
    const T r1 = f1 ? p1 : p0 + p1;
    const T r3 = f3 ? p3 : p2 + p3;
    const unsigned long long m0 = __ballot(f0), m1 = __ballot(f1), m2 = __ballot(f2), m3 = __ballot(f3);
    const int first_half = __popcll(m0) + __popcll(m1);  // run starts in slots 0 .. 127
    const int total = first_half + __popcll(m2) + __popcll(m3);
    // per half: sum of the run that is open at the end of each lane's pair, over the lanes it spans
    // (lane 0 of the second half counts as a start: nothing of that half lies below it)
    const T open0 = wave_segsum_dpp<T>(r1, f0 | f1);
    const T open1 = wave_segsum_dpp<T>(r3, f2 | f3 | (lane == 0));
    const T left = wave_readlane<T>(open0, kWave - 1);  // what the first half leaves open
    const bool joined = lanes_below(m2 | m3) == 0;      // no run starts in the second half below this lane
    const T cin0 = wave_shift_up1<T>(open0);
    const T cin1 = wave_shift_up1<T>(open1) + (joined ? left : T(0));
    int hb = lanes_below(m0) + lanes_below(m1);
    emit(f0 && hb > 0, hb - 1, cin0);
    hb += f0;
    emit(f1, hb - 1, f0 ? p0 : cin0 + p0);
    hb = first_half + lanes_below(m2) + lanes_below(m3);  // >= 1: a tile starts with a run start
    emit(f2, hb - 1, cin1);
    hb += f2;
    emit(f3, hb - 1, f2 ? p2 : cin1 + p2);
    emit(lane == kWave - 1, total - 1, joined && !(f2 | f3) ? open1 + left : open1);
    return total;
}

// The workgroup's window of x (WIDTH values from x + c0, `cnt` of them valid, the rest 0) into
// LDS: every load issued before the first LDS write (one memory round trip).
template <typename T, int WIDTH, int THREADS>
__device__ __forceinline__ void load_x_window(T *xs, const T *__restrict__ x, int64_t c0, int32_t cnt)
{
    constexpr int V = 16 / sizeof(T);           // values per 16-byte load
    constexpr int PER = WIDTH / (THREADS * V);  // loads per thread
    static_assert(PER * THREADS * V == WIDTH, "window width must be a multiple of the workgroup's loads");
    typedef T vec_t __attribute__((ext_vector_type(V)));
    vec_t buf[PER];
    const bool whole = cnt == WIDTH && ((uintptr_t)(x + c0) % 16) == 0;
    if (whole) {
#pragma unroll
        for (int k = 0; k < PER; ++k) buf[k] = reinterpret_cast<const vec_t *>(x + c0)[k * THREADS + threadIdx.x];
    } else {
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const int i0 = (k * THREADS + (int)threadIdx.x) * V;
#pragma unroll
            for (int e = 0; e < V; ++e) buf[k][e] = i0 + e < cnt ? x[c0 + i0 + e] : T(0);
        }
    }
#pragma unroll
    for (int k = 0; k < PER; ++k) reinterpret_cast<vec_t *>(xs)[k * THREADS + threadIdx.x] = buf[k];
}

}  // namespace asx
