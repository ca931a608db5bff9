// Device helpers of the id-map passes (fgl_idmap.hip): an edge's insert into the table, and what a newly numbered
// node hands to the next hop's sampling.
#pragma once
#include "fgl_common.hpp"
#include "fgl_kernels.hpp"
#include "fgl_table.hpp"

namespace fgl {

#if defined(__HIPCC__)

constexpr uint32_t kHolderBit = 0x80000000u;  // slot_of[]: the edge was the first known mention of its id when its insert ran

// find_or_insert for an edge's source id, which also says what the mark pass would otherwise have to read back
// from the table: *holder = this edge became the first known mention of the id (it installed the key, or lowered
// the key's first-edge index to its own); *displaced = the pending value it took that place from (kEmpty: none).
// An edge that became holder and is never displaced is the id's first mention.
// The probe sequence is entered at slot p with that slot's value already in hand (`s`: loaded, or returned by a
// failed compare-and-swap), so that a caller can have the first loads -- and the first compare-and-swaps -- of
// several edges in flight together before it walks any sequence further.
__device__ __forceinline__ uint32_t insert_mention_from(const TableRef t, uint32_t id, uint32_t mine, uint32_t p,
                                                        unsigned long long s, uint32_t* seen_val, bool* holder,
                                                        uint32_t* displaced)
{
    unsigned long long* slots = reinterpret_cast<unsigned long long*>(t.words);
    const unsigned long long fresh = (unsigned long long)id | ((unsigned long long)mine << 32);
    const uint32_t limit = t.mask < kMaxProbes ? t.mask + 1 : kMaxProbes;
    *holder = false;
    *displaced = kEmpty;
    for (uint32_t n = 0; n < limit; ++n) {
        if ((uint32_t)s == kEmpty) {
            const unsigned long long seen = atomicCAS(&slots[p], ~0ull, fresh);
            if (seen == ~0ull) {
                *seen_val = mine;
                *holder = true;
                return p;
            }
            s = seen;
        }
        if ((uint32_t)s == id) {
            const uint32_t v = (uint32_t)(s >> 32);
            *seen_val = v;
            if ((v & kPending) && v > mine) {
                const uint32_t old = atomicMin(&t.words[2 * (size_t)p + 1], mine);
                if (old > mine) {  // (else an even earlier mention got there between the load and the atomic)
                    *holder = true;
                    *displaced = old;
                }
            }
            return p;
        }
        p = (p + 1) & t.mask;
        s = slots[p];
    }
    return kEmpty;
}

// A node that has just been given a position in the unique list is a seed of the next hop: its row start and
// degree go to that position (store_next_hop), and its min(fanout, degree) to the next hop's per-tile edge counts.
// The two graph offsets are read by load_row_of, which callers issue early -- for every edge that may turn out to
// be a first mention -- so that the reads overlap the pass's own chain of loads.  An id outside the graph is
// marked for the next hop's sampling kernel to report.
__device__ __forceinline__ void load_row_of(const NextHop& next, int32_t id, int64_t* a, int64_t* deg)
{
    *a = kRowBadId;
    *deg = 0;
    if (id >= 0 && (int64_t)id < next.n_nodes) {
        if (next.is64) {
            const int64_t* p = static_cast<const int64_t*>(next.indptr);
            *a = p[id];
            *deg = p[id + 1] - *a;
        } else {
            const int32_t* p = static_cast<const int32_t*>(next.indptr);
            *a = p[id];
            *deg = (int64_t)p[id + 1] - *a;
        }
        if (*deg < 0) *deg = 0;
        if (*deg > 0x7FFFFFFF) *deg = 0x7FFFFFFF;
    }
}

__device__ __forceinline__ int store_next_hop(const NextHop& next, int64_t local, int64_t a, int64_t deg)
{
    next.row_start[local] = a;
    next.deg[local] = (int32_t)deg;
    return deg < next.fanout ? (int)deg : next.fanout;
}

#endif  // __HIPCC__

}  // namespace fgl
