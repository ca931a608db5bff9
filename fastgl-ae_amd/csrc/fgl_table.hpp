// The id-map's hash table: slot layout, hashing and the two probe routines, shared by the id-map
// kernels (fgl_idmap.hip) and the kernel that starts a mini-batch (fgl_blocks.hip).
//
// Slot = 8 bytes {uint32 key, uint32 val}, empty = all ones.  Slot count is a power of two,
// hash = (id * 0x9E3779B1) >> (32 - log2 slots), linear probing (8 slots per 64-byte line),
// every probe loop bounded.  Node ids are non-negative int32: no key ever equals the empty marker.
#pragma once
#include "fgl_common.hpp"

namespace fgl {

constexpr uint32_t kEmpty = 0xFFFFFFFFu;
constexpr uint32_t kDone = 0xFFFFFFFEu;  // slot_of[] marker: the edge already has its local id
constexpr uint32_t kPending = 0x80000000u;  // val = kPending | first edge index until the id is numbered
constexpr uint32_t kHashMul = 0x9E3779B1u;

struct TableRef {
    uint32_t* words;  // 2 per slot: key, val
    uint32_t mask;
    int shift;
};

inline int log2_slots(int64_t slots)
{
    int lg = 0;
    while (((int64_t)1 << lg) < slots) ++lg;
    return lg;
}

inline bool valid_slots(int64_t slots) { return slots >= 64 && slots <= ((int64_t)1 << 31) && (slots & (slots - 1)) == 0; }

inline TableRef make_ref(void* d_table, int64_t slots)
{
    TableRef t;
    t.words = static_cast<uint32_t*>(d_table);
    t.mask = (uint32_t)(slots - 1);
    t.shift = 32 - log2_slots(slots);
    return t;
}

// A probe sequence longer than this is reported as "table full" (at load <= 1/2 with this
// hash, sequences stay far below it), which also bounds the time a mis-sized table can cost.
constexpr uint32_t kMaxProbes = 4096;

// Finds the slot of `id`, inserting {id, val_if_new} if absent; if the key is already there,
// lowers its val to `val_if_new` when that is smaller (val_if_new = 0xFFFFFFFF: leave it).
// Returns kEmpty if the table is full.
//
// One 8-byte load per probe reads key and val together.  Keys only ever change from empty to a
// key and vals only ever decrease while inserts run, so an ordinary (cacheable, possibly stale)
// load is enough for the first look: a stale "empty" is settled by the 64-bit CAS, which
// installs key and val in one atomic, and a stale val can only cause a redundant atomicMin.
// *seen_val receives the val found with the key (val_if_new if this call installed the key).
// (The sequence is entered at slot p with that slot's value `s` already in hand -- loaded, or returned by a failed
// compare-and-swap -- so that a caller can put the first loads of several keys in flight before walking any further.)
__device__ __forceinline__ uint32_t find_or_insert_from(const TableRef t, uint32_t id, uint32_t val_if_new, uint32_t p,
                                                        unsigned long long s, uint32_t* seen_val)
{
    unsigned long long* slots = reinterpret_cast<unsigned long long*>(t.words);
    const unsigned long long fresh = (unsigned long long)id | ((unsigned long long)val_if_new << 32);
    const uint32_t limit = t.mask < kMaxProbes ? t.mask + 1 : kMaxProbes;
    for (uint32_t n = 0; n < limit; ++n) {
        if ((uint32_t)s == kEmpty) {
            const unsigned long long seen = atomicCAS(&slots[p], ~0ull, fresh);
            if (seen == ~0ull) {
                *seen_val = val_if_new;
                return p;
            }
            s = seen;
        }
        if ((uint32_t)s == id) {
            *seen_val = (uint32_t)(s >> 32);
            if (*seen_val > val_if_new) atomicMin(&t.words[2 * (size_t)p + 1], val_if_new);
            return p;
        }
        p = (p + 1) & t.mask;
        s = slots[p];
    }
    return kEmpty;
}

__device__ __forceinline__ uint32_t find_or_insert(const TableRef t, uint32_t id, uint32_t val_if_new, uint32_t* seen_val)
{
    const uint32_t p = (id * kHashMul) >> t.shift;
    return find_or_insert_from(t, id, val_if_new, p, reinterpret_cast<unsigned long long*>(t.words)[p], seen_val);
}

// Finds the slot of `id` without inserting.  kEmpty if absent.
__device__ __forceinline__ uint32_t find_only(const uint32_t* __restrict__ words, uint32_t mask, int shift, uint32_t id)
{
    uint32_t p = (id * kHashMul) >> shift;
    const uint32_t limit = mask < kMaxProbes ? mask + 1 : kMaxProbes;
    for (uint32_t n = 0; n < limit; ++n) {
        const uint32_t k = words[2 * (size_t)p];
        if (k == id) return p;
        if (k == kEmpty) return kEmpty;
        p = (p + 1) & mask;
    }
    return kEmpty;
}

}  // namespace fgl
