// Two probes of the memory system that the id-map's design rests on (bench.py --workload table_access):
// how fast random 8-byte loads and atomics into a table of a given size run, and whether either gets faster
// when every XCD (eighth of the chip, with an L2 of its own) works on its own eighth of the table -- and which
// XCD the workgroups of a launch land on.  No counterpart in the reference.
#include "fgl_common.hpp"
#include "fgl_kernels.hpp"

namespace fgl {

__device__ __forceinline__ uint32_t probe_mix(uint32_t x)
{
    x ^= x >> 16;
    x *= 0x7FEB352Du;
    x ^= x >> 15;
    x *= 0x846CA68Bu;
    x ^= x >> 16;
    return x;
}

// One access per lane at a pseudo-random slot.
// pattern 0: anywhere in the table; 1: inside the eighth (workgroup index % 8); 2: inside the eighth
// ((workgroup index / 8) % 8) -- the same partitioning, but not aligned with how workgroups are dealt to XCDs.
// op 0: 8-byte load; 1: 64-bit compare-and-swap of an empty slot (device scope, returning); 2: load, then the
// compare-and-swap if the slot was empty (the insert pass's pattern); 3: 32-bit add without a return value;
// 4: the compare-and-swap at workgroup scope (resolved in the XCD's L2 -- a measurement only: no kernel of the
// library communicates between workgroups that way).
__global__ __launch_bounds__(kBlock) void probe_table_access_kernel(unsigned long long* slots, int log2_slots, int pattern, int op,
                                                                    int64_t n_ops, uint32_t salt, unsigned long long* sink)
{
    const int64_t i = (int64_t)blockIdx.x * kBlock + threadIdx.x;
    if (i >= n_ops) return;
    const uint32_t w = blockIdx.x;
    const uint32_t h = probe_mix((uint32_t)i * 16u + salt * 0x9E3779B1u);
    uint32_t p;
    if (pattern == 0) {
        p = h >> (32 - log2_slots);
    } else {
        const int part_bits = log2_slots - 3;
        const uint32_t part = pattern == 1 ? (w & 7u) : ((w >> 3) & 7u);
        p = (part << part_bits) | (h >> (32 - part_bits));
    }
    unsigned long long seen = 0;
    if (op == 0) {
        seen = slots[p];
    } else if (op == 1) {
        seen = atomicCAS(&slots[p], ~0ull, (unsigned long long)i);
    } else if (op == 2) {
        seen = slots[p];
        if (seen == ~0ull) seen = atomicCAS(&slots[p], ~0ull, (unsigned long long)i);
    } else if (op == 3) {
        atomicAdd(reinterpret_cast<unsigned*>(&slots[p]), 1u);
    } else {
        unsigned long long expected = ~0ull;
        __hip_atomic_compare_exchange_strong(&slots[p], &expected, (unsigned long long)i, __ATOMIC_RELAXED, __ATOMIC_RELAXED,
                                             __HIP_MEMORY_SCOPE_WORKGROUP);
        seen = expected;
    }
    if (seen == 0x0123456789ABCDEFull) *sink = seen;  // (keeps the loads alive; no slot ever holds this value)
}

// hist[(workgroup index % 8) * 16 + XCC_ID] += 1 for every workgroup of the launch.
__global__ __launch_bounds__(kWave) void probe_xcc_kernel(uint32_t* __restrict__ hist)
{
    if (threadIdx.x != 0) return;
    const uint32_t xcc = __builtin_amdgcn_s_getreg(20 | (3 << 11)) & 15u;  // hwreg(HW_REG_XCC_ID), bits 3:0
    atomicAdd(&hist[(blockIdx.x & 7u) * 16u + xcc], 1u);
}

}  // namespace fgl

using namespace fgl;

FGL_EXPORT int fgl_probe_table_access(void* d_table, int64_t slots, int64_t n_ops, int pattern, int op, uint32_t salt,
                                      uint64_t* d_sink, void* stream)
{
    FGL_REQUIRE(d_table != nullptr && d_sink != nullptr, "probe_table_access: null pointer");
    FGL_REQUIRE(slots >= 64 && slots <= ((int64_t)1 << 31) && (slots & (slots - 1)) == 0,
                "probe_table_access: %lld slots is not a power of two in [64, 2^31]", (long long)slots);
    FGL_REQUIRE(pattern >= 0 && pattern <= 2 && op >= 0 && op <= 4, "probe_table_access: unknown pattern %d or op %d", pattern, op);
    FGL_REQUIRE(n_ops >= 0 && n_ops <= ((int64_t)1 << 31), "probe_table_access: %lld accesses outside [0, 2^31]", (long long)n_ops);
    if (n_ops == 0) return FGL_OK;
    int lg = 0;
    while (((int64_t)1 << lg) < slots) ++lg;
    hipLaunchKernelGGL(probe_table_access_kernel, dim3((unsigned)ceil_div(n_ops, kBlock)), dim3(kBlock), 0, as_stream(stream),
                       static_cast<unsigned long long*>(d_table), lg, pattern, op, n_ops, salt,
                       reinterpret_cast<unsigned long long*>(d_sink));
    FGL_CHECK_LAUNCH("probe_table_access_kernel");
    return FGL_OK;
}

FGL_EXPORT int fgl_probe_xcc_of_workgroups(uint32_t* d_hist, int n_workgroups, void* stream)
{
    FGL_REQUIRE(d_hist != nullptr, "probe_xcc_of_workgroups: null pointer");
    FGL_REQUIRE(n_workgroups >= 0 && n_workgroups <= (1 << 24), "probe_xcc_of_workgroups: %d workgroups outside [0, 2^24]", n_workgroups);
    if (n_workgroups == 0) return FGL_OK;
    hipLaunchKernelGGL(probe_xcc_kernel, dim3((unsigned)n_workgroups), dim3(kWave), 0, as_stream(stream), d_hist);
    FGL_CHECK_LAUNCH("probe_xcc_kernel");
    return FGL_OK;
}
