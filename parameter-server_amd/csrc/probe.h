// Probing of the hash array, shared by the kernel files: four lanes per key.
#pragma once

#include "table.h"

namespace pshbm {

using u32 = uint32_t;
using u64 = uint64_t;

constexpr int BLOCK = 256;  // 4 wavefronts
constexpr u32 KEYS_PER_ROUND = 16;  // keys a wavefront probes at once (four lanes each)

__device__ __forceinline__ u64 shfl64(u64 v, u32 src) {
    u32 lo = __shfl((u32)v, (int)src);
    u32 hi = __shfl((u32)(v >> 32), (int)src);
    return ((u64)hi << 32) | lo;
}


struct Found {
    u32 slot;   // where the key is, or SLOT_NONE
    u32 row;
    u32 empty;  // on a miss: the first empty slot of the bucket where the walk ended, or SLOT_NONE
};

// Four lanes (sub = 0..3 of group grp) look for `key`. Every lane of the wavefront must call
// this; lanes whose `active` is false only take part in the ballots.
__device__ __forceinline__ Found probe_find(const TableDev& t, u64 key, bool active, u32 grp,
                                            u32 sub) {
    Found f{SLOT_NONE, ROW_NONE, SLOT_NONE};
    u32 b = (u32)hash64(key) & t.bucket_mask;
    bool done = !active;
    u32 steps = 0;
    while (__ballot(!done)) {
        uint4 s = make_uint4(0u, 0u, 0u, 0u);
        if (!done) s = t.slots[(u64)b * 4 + sub];
        u64 skey = ((u64)s.y << 32) | s.x;
        bool match = !done && skey == key;
        bool empty = !done && skey == KEY_EMPTY;
        u32 m4 = (u32)(__ballot(match) >> (grp * 4)) & 0xFu;
        u32 e4 = (u32)(__ballot(empty) >> (grp * 4)) & 0xFu;
        u32 src = grp * 4 + (m4 ? (u32)__ffs((int)m4) - 1u : 0u);
        u32 row = __shfl(s.z, (int)src);
        if (!done) {
            if (m4) {
                f.slot = b * 4 + (src & 3u);
                f.row = row;
                done = true;
            } else if (e4) {
                f.empty = b * 4 + (u32)__ffs((int)e4) - 1u;
                done = true;
            } else {
                b = (b + 1) & t.bucket_mask;
                if (++steps > t.bucket_mask) done = true;
            }
        }
    }
    return f;
}

struct Located {
    u32 slot;  // slot of the key, SLOT_NONE if it is neither stored nor claimable
    u32 row;   // its row; ROW_PENDING if the slot was claimed in this launch (by this call or another)
    bool won;  // this call claimed the slot
    bool dup;  // the key was there already, or another call of this launch claimed it
};

// Four lanes (sub = 0..3 of group grp) find `key` or claim a slot for it. Every lane of the
// wavefront must call this; lanes whose `active` is false only take part in the ballots.
// need_row: also fetch the row word where the key is found by the slow path.
__device__ __forceinline__ Located find_or_claim(const TableDev& t, u64 key, bool active, u32 grp,
                                                 u32 sub, bool need_row) {
    Located r{SLOT_NONE, ROW_NONE, false, false};
    // Most keys of a batch are stored already: look for them with ordinary cached loads first.
    // What those loads show may be older than this launch, never wrong: a key that is seen is
    // stored (slots only go from empty to a key), and a key that is not seen is dealt with below.
    const Found f = probe_find(t, key, active, grp, sub);
    if (f.slot != SLOT_NONE) {
        r.slot = f.slot;
        r.row = f.row < t.max_rows ? f.row : ROW_PENDING;
        r.dup = true;
    }
    bool done = !active || f.slot != SLOT_NONE;
    u32 b = (u32)hash64(key) & t.bucket_mask;
    u32 steps = 0;
    // A key that is not seen goes straight for the first slot that looked empty. The view may be
    // old, but only in one direction (slots go from empty to a key and stay), so the first slot
    // that is truly empty is not before this one, and a copy of the key that another group stored
    // during this launch is either seen, or in this slot, or behind a slot that looked empty and
    // is not -- the compare-and-swap tells which: it finds the slot empty (claimed), holding the
    // key (a repeat), or holding another key (then the bucket is looked at again, with loads that
    // bypass the caches).
    if (__ballot(!done)) {
        const bool try_it = !done && f.empty != SLOT_NONE;
        u64 old = 0;
        if (try_it && sub == 0)
            old = atomicCAS(reinterpret_cast<unsigned long long*>(&t.slots[f.empty]),
                            (unsigned long long)KEY_EMPTY, (unsigned long long)key);
        const u64 oldb = shfl64(old, grp * 4);
        if (try_it) {
            b = f.empty >> 2;  // the buckets before it are full and stay full
            if (oldb == KEY_EMPTY || oldb == key) {
                r.slot = f.empty;
                r.row = ROW_PENDING;
                r.won = oldb == KEY_EMPTY;
                r.dup = !r.won;
                done = true;
            }
        }
    }
    while (__ballot(!done)) {
        u64 skey = 0;
        u32 srow = ROW_NONE;
        // Coherent at the device level: a slot claimed by another compute unit during this
        // launch must be seen, so the loads bypass the per-CU cache.
        if (!done) {
            uint4* sp = &t.slots[(u64)b * 4 + sub];
            skey = __hip_atomic_load(reinterpret_cast<u64*>(sp), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            if (need_row)
                srow = __hip_atomic_load(reinterpret_cast<u32*>(sp) + 2, __ATOMIC_RELAXED,
                                         __HIP_MEMORY_SCOPE_AGENT);
        }
        const bool match = !done && skey == key;
        const bool empty = !done && skey == KEY_EMPTY;
        const u32 m4 = (u32)(__ballot(match) >> (grp * 4)) & 0xFu;
        const u32 e4 = (u32)(__ballot(empty) >> (grp * 4)) & 0xFu;
        const u32 tgt = e4 ? (u32)__ffs((int)e4) - 1u : 0u;
        const bool do_cas = !done && !m4 && e4 && sub == tgt;
        u64 old = 0;
        if (do_cas)
            old = atomicCAS(reinterpret_cast<unsigned long long*>(&t.slots[(u64)b * 4 + tgt]),
                            (unsigned long long)KEY_EMPTY, (unsigned long long)key);
        const u64 oldb = shfl64(old, grp * 4 + tgt);
        const u32 msub = m4 ? (u32)__ffs((int)m4) - 1u : 0u;
        const u32 mrow = __shfl(srow, (int)(grp * 4 + msub));
        if (!done) {
            if (m4) {
                r.slot = b * 4 + msub;
                // a key that another group claimed in this launch has no row yet
                r.row = mrow < t.max_rows ? mrow : ROW_PENDING;
                r.dup = true;
                done = true;
            } else if (e4) {
                if (oldb == KEY_EMPTY) {
                    r.slot = b * 4 + tgt;
                    r.row = ROW_PENDING;
                    r.won = true;
                    done = true;
                } else if (oldb == key) {  // the same key, claimed by another group
                    r.slot = b * 4 + tgt;
                    r.row = ROW_PENDING;
                    r.dup = true;
                    done = true;
                }
                // otherwise another key took the slot: look at this bucket again
            } else {
                b = (b + 1) & t.bucket_mask;
                if (++steps > t.bucket_mask) {
                    done = true;
                    if (sub == 0) t.counters[CNT_OVERFLOW] = 1u;
                }
            }
        }
    }
    return r;
}


}  // namespace pshbm
