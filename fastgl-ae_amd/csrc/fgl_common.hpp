// Shared host/device helpers of libfastgl_hip (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include <stdio.h>
#include <string.h>

#include "fastgl_hip.h"

#define FGL_EXPORT extern "C" __attribute__((visibility("default")))

namespace fgl {

constexpr int kWave = 64;
constexpr int kBlock = 256;  // default workgroup: 4 waves

// ---- host side -------------------------------------------------------------------
void set_error(const char* fmt, ...);

#define FGL_REQUIRE(cond, ...)                 \
    do {                                       \
        if (!(cond)) {                         \
            ::fgl::set_error(__VA_ARGS__);     \
            return FGL_ERR_ARG;                \
        }                                      \
    } while (0)

#define FGL_CHECK_LAUNCH(name)                                                         \
    do {                                                                               \
        hipError_t e__ = hipGetLastError();                                            \
        if (e__ != hipSuccess) {                                                       \
            ::fgl::set_error("%s: launch failed: %s", name, hipGetErrorString(e__));   \
            return FGL_ERR_HIP;                                                        \
        }                                                                              \
    } while (0)

inline size_t align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }

// Carves sub-buffers out of a caller workspace; every piece is 256-byte aligned.
struct Carver {
    char* base;
    size_t off = 0;
    explicit Carver(void* p) : base(static_cast<char*>(p)) {}
    template <typename T>
    T* take(size_t count)
    {
        off = align_up(off, 256);
        T* p = base ? reinterpret_cast<T*>(base + off) : nullptr;
        off += count * sizeof(T);
        return p;
    }
    size_t used() const { return align_up(off, 256); }
};

inline hipStream_t as_stream(void* s) { return static_cast<hipStream_t>(s); }

// ---- device side -----------------------------------------------------------------
#if defined(__HIPCC__)

__device__ __forceinline__ int lane_id() { return (int)(threadIdx.x & (kWave - 1)); }

// actual element count of a (max, device count) pair
__device__ __forceinline__ int64_t actual_count(int64_t n_max, const int32_t* d_n)
{
    if (d_n == nullptr) return n_max;
    int64_t n = (int64_t)(*d_n);
    if (n < 0) n = 0;
    return n < n_max ? n : n_max;
}

__device__ __forceinline__ int wave_inclusive_scan(int v)
{
    const int lane = lane_id();
#pragma unroll
    for (int d = 1; d < kWave; d <<= 1) {
        int t = __shfl_up(v, d, kWave);
        if (lane >= d) v += t;
    }
    return v;
}

// Exclusive scan over a workgroup of NT threads (NT multiple of 64, <= 1024).
// `smem` needs NT/64 + 1 ints.  Returns the exclusive prefix; *total gets the block sum.
// Contains two barriers: every thread of the block must call it.
template <int NT>
__device__ __forceinline__ int block_exclusive_scan(int v, int* smem, int* total)
{
    constexpr int NW = NT / kWave;
    const int wave = (int)(threadIdx.x / kWave);
    const int incl = wave_inclusive_scan(v);
    if (lane_id() == kWave - 1) smem[wave] = incl;
    __syncthreads();
    int wave_prefix = 0, sum = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) {
        int s = smem[w];
        if (w < wave) wave_prefix += s;
        sum += s;
    }
    __syncthreads();
    *total = sum;
    return wave_prefix + incl - v;
}

// Sum of v[0..count) over a workgroup of NT threads, the same value in every thread.  `smem` needs
// NT/64 ints.  Contains two barriers: every thread of the block must call it.  Lets the workgroup
// of tile t derive its own exclusive prefix from the per-tile sums of an earlier launch, which
// saves the single-workgroup scan launch in between while the tile count is small.
template <int NT>
__device__ __forceinline__ int lane_sum_before(const int32_t* __restrict__ v, int64_t count)
{
    int s = 0;
    for (int64_t i = threadIdx.x; i < count; i += NT) s += v[i];
    return s;
}

// (lane_sum_before, then this: a caller with other loads to wait for issues those between the two, so that both
// sets are in flight together)
template <int NT>
__device__ __forceinline__ int block_sum_of_lanes(int s, int* smem)
{
    constexpr int NW = NT / kWave;
#pragma unroll
    for (int d = kWave / 2; d >= 1; d >>= 1) s += __shfl_xor(s, d, kWave);
    if (lane_id() == 0) smem[threadIdx.x / kWave] = s;
    __syncthreads();
    int sum = 0;
#pragma unroll
    for (int w = 0; w < NW; ++w) sum += smem[w];
    __syncthreads();
    return sum;
}

template <int NT>
__device__ __forceinline__ int block_sum_before(const int32_t* __restrict__ v, int64_t count, int* smem)
{
    return block_sum_of_lanes<NT>(lane_sum_before<NT>(v, count), smem);
}

// Philox4x32-10 (Salmon et al., SC'11): the counter-based generator the reference uses
// through cuRAND (sample.cu:69-70).
__device__ __forceinline__ void philox4x32_10(uint32_t c0, uint32_t c1, uint32_t c2, uint32_t c3,
                                              uint32_t k0, uint32_t k1, uint32_t out[4])
{
#pragma unroll
    for (int r = 0; r < 10; ++r) {
        const uint32_t hi0 = __umulhi(0xD2511F53u, c0), lo0 = 0xD2511F53u * c0;
        const uint32_t hi1 = __umulhi(0xCD9E8D57u, c2), lo1 = 0xCD9E8D57u * c2;
        const uint32_t n0 = hi1 ^ c1 ^ k0;
        const uint32_t n2 = hi0 ^ c3 ^ k1;
        c0 = n0; c1 = lo1; c2 = n2; c3 = lo0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    out[0] = c0; out[1] = c1; out[2] = c2; out[3] = c3;
}

#endif  // __HIPCC__

}  // namespace fgl
