// Stable LSD radix sort of (row, batch index) pairs by row: the grouping step of duplicate-key
// aggregation. The digit width is chosen per sort, 8 to 10 bits, so that keys of up to 30 bits
// take three digit passes. Every pass cuts the input into tiles of 4096 pairs, one per
// 1024-thread workgroup, and places a tile's pairs in three steps:
//   1. each of the 16 wavefronts ranks its 256 pairs, 64 at a time: one ballot per digit bit gives
//      every lane the set of lanes holding the same digit; its rank is the wave's running count for
//      that digit plus the number of lower lanes in that set (equal digits keep their input order);
//   2. thread b owns digit b: it chains the 16 wave counts into the tile's count and learns how
//      many pairs with digit b lie in earlier tiles (below);
//   3. the pairs are first put in digit order in LDS, then written out by consecutive lanes, so
//      that each run of equal digits is a contiguous, coalesced store.
// An input of one tile is sorted by one launch, all passes in LDS (sort_one_tile_kernel). Otherwise,
// how a tile learns what lies before it depends on the size of the input.
//   * Up to 256 tiles (2^20 pairs; one tile per compute unit, all resident at once) a pass is ONE
//     launch: every tile publishes its counts, the last tile of every group of 16 tiles also
//     publishes the group's count, and a tile adds up at most 15 tile words and 15 group words --
//     two batches of loads that wait only for published counts, never for another tile's finished
//     prefix, so no chain forms across the tiles. Latency matters most at this size, and one launch
//     per digit is the shortest path. The wait is bounded: if a word is not published within
//     SPIN_LIMIT polls the tile raises *err_flag and goes on with what it has, so the grid always
//     drains. The published words are read with loads that bypass the L2 (tiles run on different
//     XCDs): about 30 rows of counts per tile, more data than the tile's own pairs -- which is why
//     this scheme stops paying once tiles queue up.
//   * Above that a pass is three launches without any waiting: per-tile digit counts, a scan of
//     the counts over the tiles (which leaves in each tile's row the global position of its first
//     pair of every digit), and the placement.
#include "table.h"

namespace pshbm {

namespace {

using u32 = uint32_t;
using u64 = uint64_t;
using u16 = uint16_t;

constexpr u32 SORT_BLOCK = 1024;
constexpr u32 SORT_WAVES = SORT_BLOCK / 64;  // 16
constexpr u32 SORT_ITEMS = 4;
constexpr u32 SORT_TILE = SORT_BLOCK * SORT_ITEMS;  // 4096
constexpr u32 SORT_WAVE_SPAN = 64 * SORT_ITEMS;     // 256 pairs per wavefront
constexpr u32 MIN_BITS = 8, MAX_BITS = 10;
constexpr u32 RADIX_MAX = 1u << MAX_BITS;  // = SORT_BLOCK: a thread per digit
constexpr u32 MAX_PASSES = 4;
constexpr u32 FLAG_READY = 1u << 30, COUNT_MASK = (1u << 30) - 1u;
constexpr u32 SPIN_LIMIT = 1u << 24;
u32 g_spin_limit = SPIN_LIMIT;  // polls a tile grants a predecessor (sort_set_spin_limit)
constexpr u32 GROUP = 16;                      // tiles per group of the two-level tile prefix
constexpr u32 LOOKBACK_TILES = GROUP * GROUP;  // largest input of the one-launch passes, in tiles

constexpr u32 SEGMENTS = 16;  // three-launch passes: the tiles are cut into this many ranges

// temp layout in 32-bit words: two heads {digit totals [MAX_PASSES][SEGMENTS][RADIX_MAX], pad} used
// by alternate sorts -- each sort zeroes the other one for its successor, which saves a fill
// launch -- then rows of RADIX_MAX words: one-launch passes use, per pass, [n_tiles] tile rows and
// [n_groups] group rows; three-launch passes use [n_tiles] rows of counts, reused by every pass.
// One-launch passes keep their digit totals in segment 0. Three-launch passes keep one set of
// totals per range of tiles: 16 times fewer atomic additions meet on one word, and the scan of a
// range needs nothing from the scans of the others.
constexpr size_t HEAD_TOTALS = 0;
constexpr size_t PASS_TOTALS = (size_t)SEGMENTS * RADIX_MAX;  // words of totals per pass
constexpr size_t HEAD_WORDS = MAX_PASSES * PASS_TOTALS + 16;
constexpr size_t OFF_ROWS = 2 * HEAD_WORDS;

// The tile's four keys per thread, with the keys that became known only after the caller's
// previous launch filled in (and written back).
__device__ __forceinline__ void load_keys_late(u32* __restrict__ keys, u32 n, const SortLateKeys& late,
                                               u64 base, u32 tid, u32 (&k)[SORT_ITEMS]) {
#pragma unroll
    for (u32 j = 0; j < SORT_ITEMS; ++j) {  // all loads in flight before the first use
        const u64 i = base + (u64)j * SORT_BLOCK + tid;
        k[j] = i < n ? keys[i] : 0u;
    }
    if (late.table) {
#pragma unroll
        for (u32 j = 0; j < SORT_ITEMS; ++j) {
            const u64 i = base + (u64)j * SORT_BLOCK + tid;
            if (i < n && k[j] == late.marker) {
                k[j] = late.table[late.index[i] & 0x7FFFFFFFu].z;
                keys[i] = k[j];
            }
        }
    }
}

// One-launch passes: counts of the lowest digit over the whole input (every digit pass counts the
// next digit of the pairs it holds), and the words the passes publish start at zero.
__global__ __launch_bounds__(SORT_BLOCK) void sort_hist_kernel(u32* __restrict__ keys, u32 n,
                                                                SortLateKeys late, u32 n_tiles,
                                                                u32 passes, u32 bits,
                                                                u32* __restrict__ totals,
                                                                u32* __restrict__ status,
                                                                u32* __restrict__ next_head) {
    __shared__ u32 h[RADIX_MAX];
    const u32 tid = threadIdx.x;
    const u32 radix = 1u << bits;
    h[tid] = 0;
    const u32 tile = blockIdx.x;
    const u64 base = (u64)tile * SORT_TILE;
    u32 k[SORT_ITEMS];
    load_keys_late(keys, n, late, base, tid, k);
    __syncthreads();
#pragma unroll
    for (u32 j = 0; j < SORT_ITEMS; ++j)
        if (base + (u64)j * SORT_BLOCK + tid < n) atomicAdd(&h[k[j] & (radix - 1u)], 1u);
    __syncthreads();
    if (tid < radix) {
        if (h[tid]) atomicAdd(&totals[tid], h[tid]);
        // this tile's published words, and its group's if it opens the group
        const size_t rows = n_tiles + (n_tiles + GROUP - 1) / GROUP;
        for (u32 p = 0; p < passes; ++p) {
            status[(p * rows + tile) * RADIX_MAX + tid] = 0;
            if (tile % GROUP == 0) status[(p * rows + n_tiles + tile / GROUP) * RADIX_MAX + tid] = 0;
        }
    }
    // the totals of the NEXT sort (the other half of the head) start at zero
    for (size_t x = (size_t)tile * SORT_BLOCK + tid; x < HEAD_WORDS; x += (size_t)n_tiles * SORT_BLOCK)
        next_head[x] = 0;
}

// Three-launch passes, first launch: counts[tile][d] = pairs of the tile whose digit is d, and the
// digit totals of every range of tiles_per_seg tiles (totals[segment][d]).
__global__ __launch_bounds__(SORT_BLOCK) void sort_tile_count_kernel(u32* __restrict__ keys, u32 n,
                                                                      SortLateKeys late, u32 shift,
                                                                      u32 bits, u32 tiles_per_seg,
                                                                      u32* __restrict__ totals,
                                                                      u32* __restrict__ counts,
                                                                      u32* __restrict__ next_head) {
    __shared__ u32 h[RADIX_MAX];
    const u32 tid = threadIdx.x;
    const u32 radix = 1u << bits;
    h[tid] = 0;
    const u32 tile = blockIdx.x;
    const u64 base = (u64)tile * SORT_TILE;
    u32 k[SORT_ITEMS];
    load_keys_late(keys, n, late, base, tid, k);
    __syncthreads();
#pragma unroll
    for (u32 j = 0; j < SORT_ITEMS; ++j)
        if (base + (u64)j * SORT_BLOCK + tid < n) atomicAdd(&h[(k[j] >> shift) & (radix - 1u)], 1u);
    __syncthreads();
    if (tid < radix) {
        const u32 c = h[tid];
        counts[(size_t)tile * RADIX_MAX + tid] = c;
        if (c) atomicAdd(&totals[(size_t)(tile / tiles_per_seg) * RADIX_MAX + tid], c);
    }
    if (next_head)  // the totals of the NEXT sort (the other half of the head) start at zero
        for (size_t x = (size_t)tile * SORT_BLOCK + tid; x < HEAD_WORDS; x += (size_t)gridDim.x * SORT_BLOCK)
            next_head[x] = 0;
}

// exclusive scan over the values held by the 1024 threads of the block; all threads must call it
// (it contains a barrier). `sums` is LDS scratch of SORT_WAVES words.
__device__ __forceinline__ u32 scan_block_exclusive(u32 v, u32 tid, u32* sums) {
    const u32 lane = tid & 63u, w = tid >> 6;
    u32 incl = v;
    for (u32 off = 1; off < 64; off <<= 1) {
        const u32 o = __shfl_up(incl, off);
        if (lane >= off) incl += o;
    }
    if (lane == 63) sums[w] = incl;
    __syncthreads();
    u32 r = incl - v;
    for (u32 x = 0; x < w; ++x) r += sums[x];
    return r;
}

// Three-launch passes, second launch: counts[tile][d] becomes the position of the tile's first
// pair with digit d in the sorted output = (pairs with a smaller digit) + (pairs with digit d in
// earlier tiles). Workgroup (x, y) owns 64 digits (lane = digit, so rows are read 256 bytes at a
// time) of the y-th range of tiles, which its 16 wavefronts split into 16 consecutive parts; what
// lies before the range comes from the per-range totals.
__global__ __launch_bounds__(SORT_BLOCK) void sort_scan_kernel(u32* __restrict__ counts,
                                                                const u32* __restrict__ totals,
                                                                u32 n_tiles, u32 tiles_per_seg,
                                                                u32 radix) {
    __shared__ u32 sums[SORT_WAVES];
    __shared__ u32 dbase[64];
    __shared__ u32 part[SORT_WAVES][64];
    const u32 tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    const u32 d0 = blockIdx.x * 64u, seg = blockIdx.y;
    // pairs with a smaller digit: exclusive scan of the totals over all ranges (every workgroup
    // repeats it); pairs with this digit in earlier ranges
    u32 tot = 0, before = 0;
    if (tid < radix) {
#pragma unroll
        for (u32 x = 0; x < SEGMENTS; ++x) {
            const u32 v = totals[(size_t)x * RADIX_MAX + tid];
            tot += v;
            if (x < seg) before += v;
        }
    }
    const u32 base = scan_block_exclusive(tot, tid, sums);
    if (tid >= d0 && tid < d0 + 64u) dbase[tid - d0] = base + before;
    const u32 s0 = seg * tiles_per_seg < n_tiles ? seg * tiles_per_seg : n_tiles;
    const u32 s1 = s0 + tiles_per_seg < n_tiles ? s0 + tiles_per_seg : n_tiles;
    const u32 per = (s1 - s0 + SORT_WAVES - 1) / SORT_WAVES;
    const u32 t0 = s0 + w * per < s1 ? s0 + w * per : s1;
    const u32 t1 = t0 + per < s1 ? t0 + per : s1;
    u32* col = counts + d0 + lane;
    u32 s = 0;
    for (u32 t = t0; t < t1; t += 8) {
        u32 v[8];
#pragma unroll
        for (u32 x = 0; x < 8; ++x) v[x] = t + x < t1 ? col[(size_t)(t + x) * RADIX_MAX] : 0u;
#pragma unroll
        for (u32 x = 0; x < 8; ++x) s += v[x];
    }
    part[w][lane] = s;
    __syncthreads();
    u32 run = dbase[lane];
    for (u32 x = 0; x < w; ++x) run += part[x][lane];
    for (u32 t = t0; t < t1; t += 8) {
        u32 v[8];
#pragma unroll
        for (u32 x = 0; x < 8; ++x) v[x] = t + x < t1 ? col[(size_t)(t + x) * RADIX_MAX] : 0u;
#pragma unroll
        for (u32 x = 0; x < 8; ++x) {
            if (t + x < t1) col[(size_t)(t + x) * RADIX_MAX] = run;
            run += v[x];
        }
    }
}

// Sum of `count` (<= GROUP) published words spaced RADIX_MAX apart, starting at `words`. The loads
// are issued together; the batch is fetched again until every word carries FLAG_READY. The wait is
// bounded: past SPIN_LIMIT polls the caller gets what is there and *err_flag is raised.
__device__ __forceinline__ u32 wait_sum(const u32* words, u32 count, u32* err_flag, u32 spin_limit) {
    if (count == 0) return 0;
    if (spin_limit == 0) {  // no patience at all: the host asked for the failure path
        *err_flag = 1u;
        return 0;
    }
    u32 spins = 0;
    while (true) {
        u32 sw[GROUP];
#pragma unroll
        for (u32 q = 0; q < GROUP; ++q)
            sw[q] = q < count ? __hip_atomic_load(words + (size_t)q * RADIX_MAX, __ATOMIC_RELAXED,
                                                  __HIP_MEMORY_SCOPE_AGENT)
                              : FLAG_READY;
        u32 ready = FLAG_READY, sum = 0;
#pragma unroll
        for (u32 q = 0; q < GROUP; ++q) {
            ready &= sw[q];
            sum += sw[q] & COUNT_MASK;
        }
        if (ready & FLAG_READY) return sum;
        if (++spins > spin_limit) {  // never expected; keeps the grid from hanging
            *err_flag = 1u;
            return sum;
        }
        __builtin_amdgcn_s_sleep(2);
    }
}

// One digit pass. LOOKBACK: the one-launch scheme (totals, status, group_status, err_flag are
// used, and the counts of the next digit go to totals_next); otherwise `first_pos` is the tile's
// row of positions left by sort_scan_kernel.
template <u32 BITS, bool LOOKBACK>
__global__ __launch_bounds__(SORT_BLOCK) void sort_pass_kernel(
    const u32* __restrict__ kin, const u32* __restrict__ vin, u32* __restrict__ kout,
    u32* __restrict__ vout, u32 n, u32 shift, const u32* __restrict__ totals,
    u32* __restrict__ totals_next, u32* status, u32* group_status, const u32* __restrict__ first_pos,
    u32 n_tiles, u32* err_flag, u32 spin_limit) {
    constexpr u32 RADIX = 1u << BITS;
    // 32 KiB used twice: the per-wave digit counts (16 bits each: a wave holds 256 pairs, a tile
    // 4096) while ranking, then the tile's pairs in digit order
    __shared__ u32 pool[2 * SORT_TILE];
    __shared__ u32 hnext[LOOKBACK ? RADIX : 1];  // this tile's counts of the next digit
    __shared__ u32 binpos[RADIX];      // global position of a digit's run - its place in the tile
    __shared__ u32 tile_start[RADIX];  // place of a digit's run in the tile
    __shared__ u32 sums_a[SORT_WAVES], sums_b[SORT_WAVES];
    static_assert(SORT_WAVES * RADIX * 2 <= sizeof(pool), "wave counts must fit the pool");
    volatile u16* wcnt = reinterpret_cast<volatile u16*>(pool);  // [SORT_WAVES][RADIX]
    u32* skey = pool;
    u32* sval = pool + SORT_TILE;
    const u32 tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    // Tiles are taken in workgroup order. With the one-launch scheme every tile is resident at
    // once (at most one per compute unit), so the tiles a tile waits for are running or done;
    // should that ever not hold, the bounded spin turns a would-be hang into an error flag.
    const u32 tile = blockIdx.x;
    u32 tot = 0, gpos = 0;  // needed late; fetched with the pairs
    if (tid < RADIX) {
        if constexpr (LOOKBACK)
            tot = totals[tid];
        else
            gpos = first_pos[(size_t)tile * RADIX_MAX + tid];
    }
#pragma unroll
    for (u32 x = 0; x < SORT_WAVES * RADIX / 2 / SORT_BLOCK; ++x) pool[x * SORT_BLOCK + tid] = 0;
    if constexpr (LOOKBACK)
        if (tid < RADIX) hnext[tid] = 0;
    __syncthreads();
    const u64 tile_base = (u64)tile * SORT_TILE;
    const u64 base = tile_base + (u64)w * SORT_WAVE_SPAN;
    const u64 lt_mask = (1ull << lane) - 1ull;
    const u32 lt_lo = (u32)lt_mask, lt_hi = (u32)(lt_mask >> 32);

    u32 key[SORT_ITEMS], val[SORT_ITEMS], rnk[SORT_ITEMS];
#pragma unroll
    for (u32 j = 0; j < SORT_ITEMS; ++j) {
        const u64 i = base + (u64)j * 64 + lane;
        const bool valid = i < n;
        key[j] = valid ? kin[i] : 0xFFFFFFFFu;
        val[j] = valid ? vin[i] : 0u;
    }
    // 1. rank inside the wavefront, keeping input order among equal digits
#pragma unroll
    for (u32 j = 0; j < SORT_ITEMS; ++j) {
        const bool valid = base + (u64)j * 64 + lane < n;
        const u32 d = (key[j] >> shift) & (RADIX - 1u);
        // peers = the valid lanes that hold the same digit. Lanes past the end of the input never
        // enter the set, so the per-bit ballots need not exclude them.
        const u64 vm = __builtin_amdgcn_ballot_w64(valid);
        u32 plo = (u32)vm, phi = (u32)(vm >> 32);
#pragma unroll
        for (u32 b = 0; b < BITS; ++b) {
            const u32 bit = (d >> b) & 1u;
            const u64 m = __builtin_amdgcn_ballot_w64(bit != 0u);
            const u32 flip = bit - 1u;  // 0 where the bit is set, all ones where it is clear
            plo &= (u32)m ^ flip;
            phi &= (u32)(m >> 32) ^ flip;
        }
        const u32 before = (u32)__popc(plo & lt_lo) + (u32)__popc(phi & lt_hi);
        const u32 npeers = (u32)__popc(plo) + (u32)__popc(phi);
        u32 running = 0;
        if (valid) {
            running = wcnt[w * RADIX + d];
            if (before == 0) wcnt[w * RADIX + d] = (u16)(running + npeers);
        }
        rnk[j] = running + before;
        if constexpr (LOOKBACK)
            if (valid && totals_next) atomicAdd(&hnext[(key[j] >> (shift + BITS)) & (RADIX - 1u)], 1u);
    }
    __syncthreads();
    // 2. thread b < RADIX owns digit b: wave offsets, tile count, what lies before the tile
    u32 tile_count = 0;
    if (tid < RADIX) {
        u32 run = 0;
#pragma unroll
        for (u32 x = 0; x < SORT_WAVES; ++x) {
            const u32 c = wcnt[x * RADIX + tid];
            wcnt[x * RADIX + tid] = (u16)run;
            run += c;
        }
        tile_count = run;
        if constexpr (LOOKBACK) {
            if (totals_next && hnext[tid]) atomicAdd(&totals_next[tid], hnext[tid]);
            // publish early: successors only ever wait for these per-tile counts
            __hip_atomic_store(status + (size_t)tile * RADIX_MAX + tid, FLAG_READY | tile_count,
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
    const u32 local_start = scan_block_exclusive(tile_count, tid, sums_b);  // inside this tile
    if constexpr (LOOKBACK) {
        const u32 digit_base = scan_block_exclusive(tot, tid, sums_a);  // over the whole input
        if (tid < RADIX) {
            const u32 b = tid;
            const u32 grp = tile / GROUP, first = grp * GROUP;
            // (a) the tiles before this one in its group of GROUP: one batch of loads
            const u32 in_group = wait_sum(status + (size_t)first * RADIX_MAX + b, tile - first, err_flag, spin_limit);
            // the last tile of a group (or of the input) publishes the group's total
            if (tile + 1 == first + GROUP || tile + 1 == n_tiles)
                __hip_atomic_store(group_status + (size_t)grp * RADIX_MAX + b,
                                   FLAG_READY | ((in_group + tile_count) & COUNT_MASK), __ATOMIC_RELAXED,
                                   __HIP_MEMORY_SCOPE_AGENT);
            // (b) the groups before this one (at most GROUP - 1): one more batch
            gpos = digit_base + in_group + wait_sum(group_status + b, grp, err_flag, spin_limit);
        }
    }
    if (tid < RADIX) {
        tile_start[tid] = local_start;
        binpos[tid] = gpos - local_start;  // wraps; undone by adding the place in the tile
    }
    __syncthreads();
    // 3. digit order in LDS (over the wave counts, once every place is known), then coalesced stores
    u32 place[SORT_ITEMS];
#pragma unroll
    for (u32 j = 0; j < SORT_ITEMS; ++j) {
        const u32 d = (key[j] >> shift) & (RADIX - 1u);
        place[j] = tile_start[d] + wcnt[w * RADIX + d] + rnk[j];
    }
    __syncthreads();
#pragma unroll
    for (u32 j = 0; j < SORT_ITEMS; ++j) {
        const bool valid = base + (u64)j * 64 + lane < n;
        if (valid) {
            skey[place[j]] = key[j];
            sval[place[j]] = val[j];
        }
    }
    __syncthreads();
    const u32 tile_n = (n - tile_base) < SORT_TILE ? (u32)(n - tile_base) : SORT_TILE;
#pragma unroll
    for (u32 j = 0; j < SORT_ITEMS; ++j) {
        const u32 pl = j * SORT_BLOCK + tid;
        if (pl < tile_n) {
            const u32 k = skey[pl];
            const u32 pos = binpos[(k >> shift) & (RADIX - 1u)] + pl;
            kout[pos] = k;
            vout[pos] = sval[pl];
        }
    }
}

// An input of one tile: all digit passes in one launch. The pairs go from registers to their
// places in LDS and back, pass after pass, ranked exactly as in sort_pass_kernel; only the last
// pass writes to memory.
template <u32 BITS>
__global__ __launch_bounds__(SORT_BLOCK) void sort_one_tile_kernel(const u32* __restrict__ kin,
                                                                    const u32* __restrict__ vin,
                                                                    u32* __restrict__ kout,
                                                                    u32* __restrict__ vout, u32 n,
                                                                    u32 passes, SortLateKeys late) {
    constexpr u32 RADIX = 1u << BITS;
    __shared__ u32 pool[2 * SORT_TILE];
    __shared__ u32 tile_start[RADIX];
    __shared__ u32 sums[SORT_WAVES];
    volatile u16* wcnt = reinterpret_cast<volatile u16*>(pool);  // [SORT_WAVES][RADIX]
    u32* skey = pool;
    u32* sval = pool + SORT_TILE;
    const u32 tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    const u64 lt_mask = (1ull << lane) - 1ull;
    const u32 lt_lo = (u32)lt_mask, lt_hi = (u32)(lt_mask >> 32);
    u32 key[SORT_ITEMS], val[SORT_ITEMS], rnk[SORT_ITEMS];
#pragma unroll
    for (u32 j = 0; j < SORT_ITEMS; ++j) {
        const u32 i = w * SORT_WAVE_SPAN + j * 64 + lane;
        key[j] = i < n ? kin[i] : 0xFFFFFFFFu;
        val[j] = i < n ? vin[i] : 0u;
    }
    if (late.table) {
#pragma unroll
        for (u32 j = 0; j < SORT_ITEMS; ++j) {
            const u32 i = w * SORT_WAVE_SPAN + j * 64 + lane;
            if (i < n && key[j] == late.marker) key[j] = late.table[late.index[i] & 0x7FFFFFFFu].z;
        }
    }
    for (u32 p = 0; p < passes; ++p) {
        const u32 shift = p * BITS;
        if (p > 0) {  // the order the previous pass left in LDS
            __syncthreads();
#pragma unroll
            for (u32 j = 0; j < SORT_ITEMS; ++j) {
                const u32 i = w * SORT_WAVE_SPAN + j * 64 + lane;
                key[j] = i < n ? skey[i] : 0xFFFFFFFFu;
                val[j] = i < n ? sval[i] : 0u;
            }
            __syncthreads();
        }
#pragma unroll
        for (u32 x = 0; x < SORT_WAVES * RADIX / 2 / SORT_BLOCK; ++x) pool[x * SORT_BLOCK + tid] = 0;
        __syncthreads();
#pragma unroll
        for (u32 j = 0; j < SORT_ITEMS; ++j) {
            const bool valid = w * SORT_WAVE_SPAN + j * 64 + lane < n;
            const u32 d = (key[j] >> shift) & (RADIX - 1u);
            const u64 vm = __builtin_amdgcn_ballot_w64(valid);
            u32 plo = (u32)vm, phi = (u32)(vm >> 32);
#pragma unroll
            for (u32 b = 0; b < BITS; ++b) {
                const u32 bit = (d >> b) & 1u;
                const u64 m = __builtin_amdgcn_ballot_w64(bit != 0u);
                const u32 flip = bit - 1u;
                plo &= (u32)m ^ flip;
                phi &= (u32)(m >> 32) ^ flip;
            }
            const u32 before = (u32)__popc(plo & lt_lo) + (u32)__popc(phi & lt_hi);
            const u32 npeers = (u32)__popc(plo) + (u32)__popc(phi);
            u32 running = 0;
            if (valid) {
                running = wcnt[w * RADIX + d];
                if (before == 0) wcnt[w * RADIX + d] = (u16)(running + npeers);
            }
            rnk[j] = running + before;
        }
        __syncthreads();
        u32 tile_count = 0;
        if (tid < RADIX) {
            u32 run = 0;
#pragma unroll
            for (u32 x = 0; x < SORT_WAVES; ++x) {
                const u32 c = wcnt[x * RADIX + tid];
                wcnt[x * RADIX + tid] = (u16)run;
                run += c;
            }
            tile_count = run;
        }
        const u32 local_start = scan_block_exclusive(tile_count, tid, sums);
        if (tid < RADIX) tile_start[tid] = local_start;
        __syncthreads();
        u32 place[SORT_ITEMS];
#pragma unroll
        for (u32 j = 0; j < SORT_ITEMS; ++j) {
            const u32 d = (key[j] >> shift) & (RADIX - 1u);
            place[j] = tile_start[d] + wcnt[w * RADIX + d] + rnk[j];
        }
        __syncthreads();
        if (p + 1 < passes) {
#pragma unroll
            for (u32 j = 0; j < SORT_ITEMS; ++j)
                if (w * SORT_WAVE_SPAN + j * 64 + lane < n) {
                    skey[place[j]] = key[j];
                    sval[place[j]] = val[j];
                }
        } else {  // places of the last pass are positions of the output
#pragma unroll
            for (u32 j = 0; j < SORT_ITEMS; ++j)
                if (w * SORT_WAVE_SPAN + j * 64 + lane < n) {
                    kout[place[j]] = key[j];
                    vout[place[j]] = val[j];
                }
        }
    }
}

size_t tiles_of(size_t n) { return (n + SORT_TILE - 1) / SORT_TILE; }

template <bool LOOKBACK>
hipError_t launch_pass(u32 bits, u32 n_tiles, hipStream_t s, const u32* kin, const u32* vin, u32* kout,
                       u32* vout, u32 n, u32 shift, const u32* totals, u32* totals_next, u32* status,
                       u32* group_status, const u32* first_pos, u32* err_flag) {
    switch (bits) {
        case 8:
            sort_pass_kernel<8, LOOKBACK><<<n_tiles, SORT_BLOCK, 0, s>>>(
                kin, vin, kout, vout, n, shift, totals, totals_next, status, group_status, first_pos,
                n_tiles, err_flag, g_spin_limit);
            break;
        case 9:
            sort_pass_kernel<9, LOOKBACK><<<n_tiles, SORT_BLOCK, 0, s>>>(
                kin, vin, kout, vout, n, shift, totals, totals_next, status, group_status, first_pos,
                n_tiles, err_flag, g_spin_limit);
            break;
        case 10:
            sort_pass_kernel<10, LOOKBACK><<<n_tiles, SORT_BLOCK, 0, s>>>(
                kin, vin, kout, vout, n, shift, totals, totals_next, status, group_status, first_pos,
                n_tiles, err_flag, g_spin_limit);
            break;
        default: return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

}  // namespace

// Grows with n, so that a workspace sized for the largest batch serves every smaller one: the
// one-launch scheme of a batch of up to 2^20 pairs can need more rows than the counts of a larger one.
size_t sort_pairs_temp_bytes(size_t n) {
    const size_t n_tiles = tiles_of(n);
    const size_t lb_tiles = n_tiles < LOOKBACK_TILES ? (n_tiles ? n_tiles : 1) : LOOKBACK_TILES;
    const size_t lb_rows = MAX_PASSES * (lb_tiles + (lb_tiles + GROUP - 1) / GROUP + 1);
    const size_t rows = n_tiles > lb_rows ? n_tiles : lb_rows;
    return (OFF_ROWS + rows * RADIX_MAX) * 4;
}

size_t sort_pairs_head_bytes() { return OFF_ROWS * 4; }

void sort_set_spin_limit(uint32_t polls) { g_spin_limit = polls == ~0u ? SPIN_LIMIT : polls; }

hipError_t sort_begin(void* temp, size_t temp_bytes, unsigned parity, uint32_t* keys, size_t n,
                      unsigned end_bit, SortPlan* plan, hipStream_t s, const SortLateKeys* late) {
    plan->n = 0;
    plan->passes = 0;
    if (n == 0) return hipSuccess;
    if (n > COUNT_MASK || temp_bytes < sort_pairs_temp_bytes(n)) return hipErrorInvalidValue;
    if (end_bit == 0 || end_bit > 32) return hipErrorInvalidValue;
    // as few passes as 10-bit digits allow, then the narrowest digit that still covers the key
    const u32 passes = (end_bit + MAX_BITS - 1) / MAX_BITS;
    u32 bits = (end_bit + passes - 1) / passes;
    if (bits < MIN_BITS) bits = MIN_BITS;
    if (passes > MAX_PASSES) return hipErrorInvalidValue;
    const u32 n_tiles = (u32)tiles_of(n);
    u32* words = static_cast<u32*>(temp);
    u32* head = words + (parity & 1u) * HEAD_WORDS;
    u32* next_head = words + ((parity & 1u) ^ 1u) * HEAD_WORDS;
    plan->n = (u32)n;
    plan->n_tiles = n_tiles;
    plan->passes = passes;
    plan->digit_passes = passes;
    plan->bits = bits;
    plan->one_tile = n_tiles == 1;
    plan->uses_head = !plan->one_tile;
    plan->late = SortLateKeys{0u, nullptr, nullptr};
    if (late) plan->late = *late;
    if (plan->one_tile) {  // everything happens in the one sort_pass call
        plan->passes = 1;
        plan->lookback = false;
        plan->totals = nullptr;
        plan->status = nullptr;
        plan->rows = 0;
        return hipSuccess;
    }
    plan->lookback = n_tiles <= LOOKBACK_TILES;
    plan->totals = head + HEAD_TOTALS;
    plan->status = words + OFF_ROWS;
    plan->rows = n_tiles + (n_tiles + GROUP - 1) / GROUP;  // one-launch passes: tile and group rows
    SortLateKeys lk{0u, nullptr, nullptr};
    if (late) lk = *late;
    if (plan->lookback)
        sort_hist_kernel<<<n_tiles, SORT_BLOCK, 0, s>>>(keys, (u32)n, lk, n_tiles, passes, bits,
                                                        plan->totals, plan->status, next_head);
    else
        sort_tile_count_kernel<<<n_tiles, SORT_BLOCK, 0, s>>>(keys, (u32)n, lk, 0u, bits,
                                                              (n_tiles + SEGMENTS - 1) / SEGMENTS,
                                                              plan->totals, plan->status, next_head);
    return hipGetLastError();
}

hipError_t sort_pass(const SortPlan& plan, unsigned p, const uint32_t* kin, const uint32_t* vin,
                     uint32_t* kout, uint32_t* vout, uint32_t* err_flag, hipStream_t s) {
    if (plan.n == 0) return hipSuccess;
    if (p >= plan.passes) return hipErrorInvalidValue;
    if (plan.one_tile) {
        switch (plan.bits) {
            case 8:
                sort_one_tile_kernel<8><<<1, SORT_BLOCK, 0, s>>>(kin, vin, kout, vout, plan.n,
                                                                 plan.digit_passes, plan.late);
                break;
            case 9:
                sort_one_tile_kernel<9><<<1, SORT_BLOCK, 0, s>>>(kin, vin, kout, vout, plan.n,
                                                                 plan.digit_passes, plan.late);
                break;
            case 10:
                sort_one_tile_kernel<10><<<1, SORT_BLOCK, 0, s>>>(kin, vin, kout, vout, plan.n,
                                                                  plan.digit_passes, plan.late);
                break;
            default: return hipErrorInvalidValue;
        }
        return hipGetLastError();
    }
    const u32 shift = plan.bits * p;
    u32* totals = plan.totals + p * PASS_TOTALS;
    if (plan.lookback) {
        u32* totals_next = p + 1 < plan.passes ? plan.totals + (p + 1) * PASS_TOTALS : nullptr;
        u32* status = plan.status + (size_t)p * plan.rows * RADIX_MAX;
        u32* group_status = plan.status + ((size_t)p * plan.rows + plan.n_tiles) * RADIX_MAX;
        return launch_pass<true>(plan.bits, plan.n_tiles, s, kin, vin, kout, vout, plan.n, shift, totals,
                                 totals_next, status, group_status, nullptr, err_flag);
    }
    const SortLateKeys none{0u, nullptr, nullptr};
    const u32 tiles_per_seg = (plan.n_tiles + SEGMENTS - 1) / SEGMENTS;
    if (p > 0) {  // pass 0 was counted by sort_begin
        sort_tile_count_kernel<<<plan.n_tiles, SORT_BLOCK, 0, s>>>(const_cast<u32*>(kin), plan.n, none,
                                                                   shift, plan.bits, tiles_per_seg,
                                                                   totals, plan.status, nullptr);
        hipError_t e = hipGetLastError();
        if (e != hipSuccess) return e;
    }
    const u32 radix = 1u << plan.bits;
    sort_scan_kernel<<<dim3(radix / 64, SEGMENTS), SORT_BLOCK, 0, s>>>(plan.status, totals, plan.n_tiles,
                                                                       tiles_per_seg, radix);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    return launch_pass<false>(plan.bits, plan.n_tiles, s, kin, vin, kout, vout, plan.n, shift, nullptr,
                              nullptr, nullptr, nullptr, plan.status, err_flag);
}

hipError_t sort_pairs(void* temp, size_t temp_bytes, unsigned parity, uint32_t* keys_a,
                      uint32_t* keys_b, uint32_t* vals_a, uint32_t* vals_b, size_t n,
                      unsigned end_bit, bool* result_in_b, uint32_t* err_flag, hipStream_t s) {
    *result_in_b = false;
    SortPlan plan;
    hipError_t e = sort_begin(temp, temp_bytes, parity, keys_a, n, end_bit, &plan, s);
    if (e != hipSuccess) return e;
    u32 *kin = keys_a, *vin = vals_a, *kout = keys_b, *vout = vals_b;
    for (u32 p = 0; p < plan.passes; ++p) {
        e = sort_pass(plan, p, kin, vin, kout, vout, err_flag, s);
        if (e != hipSuccess) return e;
        u32* tk = kin;
        u32* tv = vin;
        kin = kout;
        vin = vout;
        kout = tk;
        vout = tv;
    }
    *result_in_b = (plan.passes & 1u) != 0;
    return hipSuccess;
}

}  // namespace pshbm
