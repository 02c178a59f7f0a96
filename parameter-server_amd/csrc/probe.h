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

}  // namespace pshbm
