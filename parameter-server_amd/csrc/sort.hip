// Stable LSD radix sort of (slot, batch index) pairs by slot: the grouping step of duplicate-key
// aggregation. Written for batches of 10^5..10^7 pairs, where launch count and latency matter more
// than bandwidth: one histogram launch, then ONE launch per 8-bit digit.
//
// A digit pass cuts the input into tiles of 4096 pairs, one per 1024-thread workgroup:
//   1. each of the 16 wavefronts ranks its 256 pairs, 64 at a time: eight ballots give every lane
//      the set of lanes holding the same digit; its rank is the wave's running count for that
//      digit plus the number of lower lanes in that set (equal digits keep their input order);
//   2. thread b < 256 owns digit b: it chains the 16 wave counts into the tile count and publishes
//      it; the last tile of every group of 16 tiles also publishes the group's count. The number
//      of pairs with digit b in earlier tiles is then the sum of at most 15 tile words and of the
//      group words before -- two or three batches of loads that wait only for published counts,
//      never for another tile's finished prefix, so no chain forms across the tiles;
//   3. the pairs are first put in digit order in LDS, then written out by consecutive lanes, so
//      that each run of equal digits is a contiguous, coalesced store.
// The wait is bounded: if a word is not published within SPIN_LIMIT polls the tile raises
// *err_flag and goes on with what it has, so the grid always drains.
#include "table.h"

namespace pshbm {

namespace {

using u32 = uint32_t;
using u64 = uint64_t;

constexpr u32 SORT_BLOCK = 1024;
constexpr u32 SORT_WAVES = SORT_BLOCK / 64;  // 16
constexpr u32 SORT_ITEMS = 4;
constexpr u32 SORT_TILE = SORT_BLOCK * SORT_ITEMS;  // 4096
constexpr u32 SORT_WAVE_SPAN = 64 * SORT_ITEMS;     // 256 pairs per wavefront
constexpr u32 RADIX = 256;
constexpr u32 MAX_PASSES = 4;
constexpr u32 FLAG_READY = 1u << 30, COUNT_MASK = (1u << 30) - 1u;
constexpr u32 SPIN_LIMIT = 1u << 24;
constexpr u32 GROUP = 16;  // tiles per group of the two-level tile prefix

// temp layout in 32-bit words: two heads {digit totals [MAX_PASSES][RADIX], tile counters
// [MAX_PASSES] (+ pad)} used by alternate sorts -- each sort zeroes the other one for its
// successor, which saves a fill launch -- then, per pass, [n_tiles][RADIX] tile words and
// [n_groups][RADIX] group words.
constexpr size_t HEAD_TOTALS = 0;
constexpr size_t HEAD_COUNTERS = MAX_PASSES * RADIX;
constexpr size_t HEAD_WORDS = HEAD_COUNTERS + 16;
constexpr size_t OFF_STATUS = 2 * HEAD_WORDS;

__global__ __launch_bounds__(SORT_BLOCK) void sort_hist_kernel(u32* __restrict__ keys, u32 n,
                                                                SortLateKeys late, u32 n_tiles,
                                                                u32 passes,
                                                                u32* __restrict__ totals,
                                                                u32* __restrict__ status,
                                                                u32* __restrict__ next_head) {
    // Counts the lowest digit only; every digit pass counts the next digit of the pairs it holds.
    __shared__ u32 h[RADIX];
    const u32 tid = threadIdx.x;
    if (tid < RADIX) h[tid] = 0;
    const u32 tile = blockIdx.x;
    const u64 base = (u64)tile * SORT_TILE;
    u32 k[SORT_ITEMS];
#pragma unroll
    for (u32 j = 0; j < SORT_ITEMS; ++j) {  // all loads in flight before the first LDS atomic
        const u64 i = base + (u64)j * SORT_BLOCK + tid;
        k[j] = i < n ? keys[i] : 0u;
    }
    if (late.table) {  // keys that became known only after the caller's previous launch
#pragma unroll
        for (u32 j = 0; j < SORT_ITEMS; ++j) {
            const u64 i = base + (u64)j * SORT_BLOCK + tid;
            if (i < n && k[j] == late.marker) {
                k[j] = late.table[late.index[i] & 0x7FFFFFFFu].z;
                keys[i] = k[j];
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (u32 j = 0; j < SORT_ITEMS; ++j)
        if (base + (u64)j * SORT_BLOCK + tid < n) atomicAdd(&h[k[j] & 255u], 1u);
    __syncthreads();
    {
        const u32 p = tid >> 8, b = tid & 255u;  // 1024 threads = MAX_PASSES x RADIX
        if (p == 0 && h[b]) atomicAdd(&totals[b], h[b]);
        if (p < passes) {  // this tile's published words, and its group's if it opens the group
            const size_t rows = n_tiles + (n_tiles + GROUP - 1) / GROUP;
            status[(p * rows + tile) * RADIX + b] = 0;
            if (tile % GROUP == 0) status[(p * rows + n_tiles + tile / GROUP) * RADIX + b] = 0;
        }
    }
    // the totals and tile counters of the NEXT sort (the other half of the head) start at zero
    if (tile == 0)
        for (u32 x = tid; x < HEAD_WORDS; x += SORT_BLOCK) next_head[x] = 0;
}

// exclusive scan over the 256 values held by threads 0..255 (4 wavefronts); all threads of the
// block must call it (it contains a barrier). `sums` is LDS scratch of 4 words.
__device__ __forceinline__ u32 scan256_exclusive(u32 v, u32 tid, u32* sums) {
    const u32 lane = tid & 63u, w = tid >> 6;
    u32 incl = v;
    for (u32 off = 1; off < 64; off <<= 1) {
        const u32 o = __shfl_up(incl, off);
        if (lane >= off) incl += o;
    }
    if (lane == 63 && w < 4) sums[w] = incl;
    __syncthreads();
    u32 r = incl - v;
    for (u32 x = 0; x < w && x < 4; ++x) r += sums[x];
    return r;
}

// Sum of `count` (<= GROUP) published words spaced RADIX apart, starting at `words`. The loads of a
// batch are issued together; the batch is fetched again until every word carries FLAG_READY. The
// wait is bounded: past SPIN_LIMIT polls the caller gets what is there and *err_flag is raised.
__device__ __forceinline__ u32 wait_sum(const u32* words, u32 count, u32* err_flag) {
    if (count == 0) return 0;
    u32 spins = 0;
    while (true) {
        u32 sw[GROUP];
#pragma unroll
        for (u32 q = 0; q < GROUP; ++q)
            sw[q] = q < count ? __hip_atomic_load(words + (size_t)q * RADIX, __ATOMIC_RELAXED,
                                                  __HIP_MEMORY_SCOPE_AGENT)
                              : FLAG_READY;
        u32 ready = FLAG_READY, sum = 0;
#pragma unroll
        for (u32 q = 0; q < GROUP; ++q) {
            ready &= sw[q];
            sum += sw[q] & COUNT_MASK;
        }
        if (ready & FLAG_READY) return sum;
        if (++spins > SPIN_LIMIT) {  // never expected; keeps the grid from hanging
            *err_flag = 1u;
            return sum;
        }
        __builtin_amdgcn_s_sleep(1);
    }
}

__global__ __launch_bounds__(SORT_BLOCK) void sort_pass_kernel(
    const u32* __restrict__ kin, const u32* __restrict__ vin, u32* __restrict__ kout,
    u32* __restrict__ vout, u32 n, u32 shift, const u32* __restrict__ totals,
    u32* __restrict__ totals_next, u32* status, u32* group_status, u32 n_tiles, u32* err_flag) {
    __shared__ volatile u32 wcnt[SORT_WAVES][RADIX];  // per-wave digit counts, then offsets
    __shared__ u32 hnext[RADIX];                      // this tile's counts of the next digit
    __shared__ u32 binpos[RADIX];                     // global position of a digit's run - its place in the tile
    __shared__ u32 tile_start[RADIX];                 // place of a digit's run in the tile
    __shared__ u32 skey[SORT_TILE], sval[SORT_TILE];
    __shared__ u32 sums_a[4], sums_b[4];
    const u32 tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    // Tiles are taken in workgroup order. The hardware starts workgroups in that order, so a
    // tile's predecessors are running (or done) when it looks back; should that ever not hold,
    // the bounded spin below turns a would-be hang into an error flag.
    const u32 tile = blockIdx.x;
    const u32 tot = tid < RADIX ? totals[tid] : 0u;  // needed late; fetched with the pairs
#pragma unroll
    for (u32 x = 0; x < SORT_WAVES * RADIX / SORT_BLOCK; ++x)
        (&wcnt[0][0])[x * SORT_BLOCK + tid] = 0;
    if (tid < RADIX) hnext[tid] = 0;
    __syncthreads();
    const u64 tile_base = (u64)tile * SORT_TILE;
    const u64 base = tile_base + (u64)w * SORT_WAVE_SPAN;
    const u64 lt_mask = (1ull << lane) - 1ull;

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
        const u32 d = (key[j] >> shift) & 255u;
        u64 peers = __ballot(valid);
#pragma unroll
        for (u32 b = 0; b < 8; ++b) {
            const bool bit = (d >> b) & 1u;
            const u64 m = __ballot(valid && bit);
            peers &= bit ? m : ~m;
        }
        const u32 before = (u32)__popcll(peers & lt_mask);
        u32 running = 0;
        if (valid) {
            running = wcnt[w][d];
            if (before == 0) wcnt[w][d] = running + (u32)__popcll(peers);
        }
        rnk[j] = running + before;
        if (valid && totals_next) atomicAdd(&hnext[(key[j] >> (shift + 8)) & 255u], 1u);
    }
    __syncthreads();
    // 2. thread b < 256 owns digit b: wave offsets, tile count, digit base, look-back
    u32 tile_count = 0;
    if (tid < RADIX) {
        u32 run = 0;
#pragma unroll
        for (u32 x = 0; x < SORT_WAVES; ++x) {
            const u32 c = wcnt[x][tid];
            wcnt[x][tid] = run;
            run += c;
        }
        tile_count = run;
        if (totals_next && hnext[tid]) atomicAdd(&totals_next[tid], hnext[tid]);
        // publish early: successors only ever wait for these per-tile counts
        __hip_atomic_store(status + (size_t)tile * RADIX + tid, FLAG_READY | tile_count,
                           __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    const u32 digit_base = scan256_exclusive(tot, tid, sums_a);       // over the whole input
    const u32 local_start = scan256_exclusive(tile_count, tid, sums_b);  // inside this tile
    if (tid < RADIX) {
        const u32 b = tid;
        const u32 grp = tile / GROUP, first = grp * GROUP;
        // (a) the tiles before this one in its group of GROUP: one batch of loads
        const u32 in_group = wait_sum(status + (size_t)first * RADIX + b, tile - first, err_flag);
        // the last tile of a group (or of the input) publishes the group's total
        if (tile + 1 == first + GROUP || tile + 1 == n_tiles)
            __hip_atomic_store(group_status + (size_t)grp * RADIX + b,
                               FLAG_READY | ((in_group + tile_count) & COUNT_MASK), __ATOMIC_RELAXED,
                               __HIP_MEMORY_SCOPE_AGENT);
        // (b) the groups before this one, GROUP words per round trip
        u32 excl = in_group;
        for (u32 g0 = 0; g0 < grp; g0 += GROUP)
            excl += wait_sum(group_status + (size_t)g0 * RADIX + b, (grp - g0) < GROUP ? grp - g0 : GROUP,
                             err_flag);
        tile_start[b] = local_start;
        binpos[b] = digit_base + excl - local_start;  // wraps; undone by adding the place in the tile
    }
    __syncthreads();
    // 3. digit order in LDS, then coalesced stores
#pragma unroll
    for (u32 j = 0; j < SORT_ITEMS; ++j) {
        const bool valid = base + (u64)j * 64 + lane < n;
        if (valid) {
            const u32 d = (key[j] >> shift) & 255u;
            const u32 place = tile_start[d] + wcnt[w][d] + rnk[j];
            skey[place] = key[j];
            sval[place] = val[j];
        }
    }
    __syncthreads();
    const u32 tile_n = (n - tile_base) < SORT_TILE ? (u32)(n - tile_base) : SORT_TILE;
#pragma unroll
    for (u32 j = 0; j < SORT_ITEMS; ++j) {
        const u32 place = j * SORT_BLOCK + tid;
        if (place < tile_n) {
            const u32 k = skey[place];
            const u32 pos = binpos[(k >> shift) & 255u] + place;
            kout[pos] = k;
            vout[pos] = sval[place];
        }
    }
}

}  // namespace

size_t sort_pairs_temp_bytes(size_t n) {
    const size_t n_tiles = (n + SORT_TILE - 1) / SORT_TILE;
    const size_t rows = (n_tiles ? n_tiles : 1) + (n_tiles + GROUP - 1) / GROUP + 1;
    return (OFF_STATUS + (size_t)MAX_PASSES * rows * RADIX) * 4;
}

size_t sort_pairs_head_bytes() { return OFF_STATUS * 4; }

hipError_t sort_begin(void* temp, size_t temp_bytes, unsigned parity, uint32_t* keys, size_t n,
                      unsigned end_bit, SortPlan* plan, hipStream_t s, const SortLateKeys* late) {
    plan->n = 0;
    plan->passes = 0;
    if (n == 0) return hipSuccess;
    if (n > COUNT_MASK || temp_bytes < sort_pairs_temp_bytes(n)) return hipErrorInvalidValue;
    const u32 passes = (end_bit + 7) / 8;
    if (passes == 0 || passes > MAX_PASSES) return hipErrorInvalidValue;
    const u32 n_tiles = (u32)((n + SORT_TILE - 1) / SORT_TILE);
    u32* words = static_cast<u32*>(temp);
    u32* head = words + (parity & 1u) * HEAD_WORDS;
    u32* next_head = words + ((parity & 1u) ^ 1u) * HEAD_WORDS;
    plan->n = (u32)n;
    plan->n_tiles = n_tiles;
    plan->passes = passes;
    plan->totals = head + HEAD_TOTALS;
    plan->status = words + OFF_STATUS;
    plan->rows = n_tiles + (n_tiles + GROUP - 1) / GROUP;  // per pass: tile words, group words
    SortLateKeys lk{0u, nullptr, nullptr};
    if (late) lk = *late;
    sort_hist_kernel<<<n_tiles, SORT_BLOCK, 0, s>>>(keys, (u32)n, lk, n_tiles, passes, plan->totals,
                                                    plan->status, next_head);
    return hipGetLastError();
}

hipError_t sort_pass(const SortPlan& plan, unsigned p, const uint32_t* kin, const uint32_t* vin,
                     uint32_t* kout, uint32_t* vout, uint32_t* err_flag, hipStream_t s) {
    if (plan.n == 0) return hipSuccess;
    if (p >= plan.passes) return hipErrorInvalidValue;
    sort_pass_kernel<<<plan.n_tiles, SORT_BLOCK, 0, s>>>(
        kin, vin, kout, vout, plan.n, 8 * p, plan.totals + p * RADIX,
        p + 1 < plan.passes ? plan.totals + (p + 1) * RADIX : nullptr,
        plan.status + (size_t)p * plan.rows * RADIX,
        plan.status + ((size_t)p * plan.rows + plan.n_tiles) * RADIX, plan.n_tiles, err_flag);
    return hipGetLastError();
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
