// The partitioned push: duplicate-key aggregation and row update of a large batch without a global
// sort (the duplicate merge of pico-ps/operator/SparsePushOperator.h:134-141 and the per-item loop
// of :245-268).
//
// The batch is cut into tiles of 4096 keys and the key space into P partitions, a partition being a
// range of home buckets of the hash array. Three launches:
//   1. part_tile_kernel     a workgroup per tile: finds the keys that repeat inside the tile (a hash
//                           table in LDS), adds up their gradient rows into one pre-summed row per
//                           key, and leaves one entry {key, reference, row handle} per distinct key of the tile,
//                           grouped by partition, in the tile's staging block, with the place where
//                           each partition's entries start in the block; a reference is the batch
//                           index of the gradient row or the number of a pre-summed row.
//   2. part_apply_kernel    a workgroup per partition: collects the partition's entries from the
//                           staging blocks of all tiles (the tiles' start words of its partition and
//                           of the next give every segment, and their sum the number of entries in
//                           lower partitions: no scan launch, no copy into partition order), groups
//                           them by key (LDS hash table again; a key has at most one entry per tile,
//                           so the hottest key of a batch is a list of a few hundred references, not
//                           of a hundred thousand), probes the table ONCE per distinct key, adds up
//                           each key's rows and takes the optimizer step. A key that is not stored
//                           claims a slot; its summed gradient is parked for the last launch.
//   3. part_insert_kernel   numbers the new keys densely (prefix over the partitions' counts),
//                           initialises their rows and takes their step.
// Sums are accumulated in double precision and rounded to fp32 once per tile and once per key: the
// result does not depend on the order in which a key's rows are met beyond the last bit of a
// 53-bit sum. Loads that a later step needs are never put behind a branch (a lane without work
// loads element 0 and drops it): the compiler then keeps all of them in flight together, which
// is what these latency-bound kernels live on.
#include "table.h"
#include "probe.h"
#include "rowops.h"

namespace pshbm {

namespace {

using u16 = uint16_t;

constexpr u32 PT_TILE = 4096, PT_BLOCK = 1024, PT_ITEMS = PT_TILE / PT_BLOCK;
constexpr u32 PT_HT = 2 * PT_TILE;            // slots of a tile's LDS hash table
constexpr u32 PT_MAX_MULTI = PT_TILE / 2;     // pre-summed rows a tile can produce
// accumulators: the room of the tile's key array, of its hash table and of half its counts (72 KiB)
constexpr u32 PT_ACC_DOUBLES = (PT_TILE * 8 + PT_HT * 4 + (PT_TILE - PT_MAX_MULTI) * 4) / 8;
constexpr u32 REF_PSUM = 0x80000000u;         // reference to a pre-summed row
constexpr u32 NONE32 = 0xFFFFFFFFu;
constexpr u32 PA_BLOCK = 512, PA_ITEMS = 4, PA_CAP = PA_BLOCK * PA_ITEMS;  // entries a partition pass holds
constexpr u32 PA_HT = 2 * PA_CAP;
// entries a partition should hold on average: short rows / longer ones (whose list sums take a
// round of LDS accumulators per 2048 / dim lists, so that fuller partitions cost them rounds)
constexpr double PART_TARGET = 1250.0, PART_TARGET_LONG_ROWS = 625.0;
constexpr u32 PA_ACC_DOUBLES = PA_HT / 2;     // the room of the partition's hash table (16 KiB)
constexpr u32 AUX_NEW = 0x80000000u;     // in a distinct key's aux word: the key claimed a slot in this launch
constexpr u32 AUX_SINGLE = 0x40000000u;  // the key has one entry (low 16 bits: where its reference lies)
constexpr u32 ROW_WALK = 0xFFFFFFFDu;    // in a distinct key's row word: still to be looked up by the walk
constexpr u32 AUX_MULTI_MASK = 0x3FFFu;  // bits 16..29 of a key with several entries: its list number

// exclusive scan over the NT threads of the block (64-bit packed fields); all threads call it
template <u32 NT>
__device__ __forceinline__ u64 block_scan_excl(u64 v, u32 tid, u64* sums, u64* total) {
    const u32 lane = tid & 63u, w = tid >> 6;
    u64 incl = v;
    for (u32 off = 1; off < 64; off <<= 1) {
        const u64 o = shfl64(incl, (lane >= off) ? lane - off : lane);
        if (lane >= off) incl += o;
    }
    if (lane == 63) sums[w] = incl;
    __syncthreads();
    u64 before = 0, all = 0;
    for (u32 x = 0; x < NT / 64; ++x) {
        const u64 c = sums[x];
        if (x < w) before += c;
        all += c;
    }
    *total = all;
    __syncthreads();
    return before + incl - v;
}

// Item q (key lkey[q], hash h) finds the item that stands for its key -- the first one to claim
// the key's slot of the LDS hash table -- and its arrival number among the items of that key.
__device__ __forceinline__ void dedupe_insert(u64 key, u32 q, u64 h, const u64* lkey, u32* owner, u32* cnt,
                                              u32 ht_mask, u32& rep, u32& arrival) {
    u32 s = (u32)(h >> 40) & ht_mask;
    while (true) {
        const u32 old = atomicCAS(&owner[s], NONE32, q);
        if (old == NONE32) {
            rep = q;
            break;
        }
        if (lkey[old] == key) {
            rep = old;
            break;
        }
        s = (s + 1) & ht_mask;
    }
    arrival = atomicAdd(&cnt[rep], 1u);
}

// The same with the count kept in the table's word: owner[s] = item | arrivals << 16 (at most 2^15
// items). `slot` is where the key's word lies, for the count to be read later.
__device__ __forceinline__ void dedupe_insert_packed(u64 key, u32 q, u64 h, const u64* lkey, u32* owner,
                                                     u32 ht_mask, u32& rep, u32& arrival, u32& slot) {
    u32 s = (u32)(h >> 40) & ht_mask;
    while (true) {
        const u32 old = atomicCAS(&owner[s], NONE32, q | (1u << 16));
        if (old == NONE32) {
            rep = q;
            arrival = 0;
            break;
        }
        if (lkey[old & 0xFFFFu] == key) {
            rep = old & 0xFFFFu;
            arrival = atomicAdd(&owner[s], 1u << 16) >> 16;
            break;
        }
        s = (s + 1) & ht_mask;
    }
    slot = s;
}

template <typename T>
struct Acc;
template <>
struct Acc<float> {
    double a;
    __device__ __forceinline__ void zero() { a = 0.0; }
    __device__ __forceinline__ void add(float v) { a += (double)v; }
    __device__ __forceinline__ void flush(double* p) const { atomicAdd(p, a); }
    __device__ __forceinline__ static float load(const double* p) { return (float)p[0]; }
};
template <>
struct Acc<float4> {
    double a, b, c, d;
    __device__ __forceinline__ void zero() { a = b = c = d = 0.0; }
    __device__ __forceinline__ void add(float4 v) {
        a += (double)v.x;
        b += (double)v.y;
        c += (double)v.z;
        d += (double)v.w;
    }
    __device__ __forceinline__ void flush(double* p) const {
        atomicAdd(p, a);
        atomicAdd(p + 1, b);
        atomicAdd(p + 2, c);
        atomicAdd(p + 3, d);
    }
    __device__ __forceinline__ static float4 load(const double* p) {
        return make_float4((float)p[0], (float)p[1], (float)p[2], (float)p[3]);
    }
};

// Sums of lists of gradient rows, all lists at once: elements [lo, hi) are cut into equal runs, one
// per lane group (so a long list is spread over several groups), element e belongs to list lid[e]
// (ascending in e) and its row is src(e); a group adds consecutive elements of one list in
// registers and adds the sum to the list's accumulators in LDS when the list changes.
// acc[((list - list_base) * units + c) * N + x], double, zero on entry.
template <typename T>
struct ListSum {
    Acc<T> a;
    u32 cur, list_base, units, c;
    double* acc;
    __device__ __forceinline__ void begin(double* acc_, u32 list_base_, u32 units_, u32 c_) {
        acc = acc_;
        list_base = list_base_;
        units = units_;
        c = c_;
        cur = NONE32;
        a.zero();
    }
    __device__ __forceinline__ void flush() {
        if (cur != NONE32) a.flush(acc + ((size_t)(cur - list_base) * units + c) * (sizeof(T) / 4));
    }
    __device__ __forceinline__ void take(u32 l, T v) {
        if (l != cur) {
            flush();
            cur = l;
            a.zero();
        }
        a.add(v);
    }
};

// elements first, first + 1, ... below last
template <typename T, typename SRC>
__device__ __forceinline__ void flat_sum_from(SRC src, const u16* lid, u32 first, u32 last, u32 c, ListSum<T>& ls) {
    u32 e = first;
    for (; e + 3 < last; e += 4) {  // four rows in flight
        const u32 l0 = lid[e], l1 = lid[e + 1], l2 = lid[e + 2], l3 = lid[e + 3];
        const T v0 = src(e)[c], v1 = src(e + 1)[c], v2 = src(e + 2)[c], v3 = src(e + 3)[c];
        ls.take(l0, v0);
        ls.take(l1, v1);
        ls.take(l2, v2);
        ls.take(l3, v3);
    }
    for (; e < last; ++e) ls.take(lid[e], src(e)[c]);
}

// Lane group g of NG takes the g-th of NG equal runs of consecutive elements: consecutive elements
// mostly belong to one list, so a group adds to the accumulators about once per list it meets and
// not once per element (additions of doubles in LDS go one lane at a time).
__device__ __forceinline__ u32 chunk_len(u32 lo, u32 hi, u32 NG) { return (hi - lo + NG - 1) / NG; }

template <typename T, typename SRC>
__device__ __forceinline__ void flat_sum(SRC src, const u16* lid, u32 lo, u32 hi, u32 list_base, double* acc,
                                         u32 units, u32 NG, u32 g, u32 c) {
    ListSum<T> ls;
    ls.begin(acc, list_base, units, c);
    const u32 len = chunk_len(lo, hi, NG);
    const u32 first = lo + g * len < hi ? lo + g * len : hi;
    const u32 last = first + len < hi ? first + len : hi;
    flat_sum_from<T>(src, lid, first, last, c, ls);
    ls.flush();
}

__device__ __forceinline__ u32 partition_of(const TableDev& t, u64 h, u32 part_shift) {
    return ((u32)h & t.bucket_mask) >> part_shift;
}

// ---- 1. tile kernel ---------------------------------------------------------------------------
// LDS (dynamic, 112 KiB + a word per partition): keys of the tile (later the accumulators) | hash table (later the list of
// keys that repeat) | per-item counts | per-item aux | list of repeating items + their list numbers |
// partition histogram.
constexpr u32 PT_OFF_OWNER = PT_TILE * 8;
constexpr u32 PT_OFF_CNT = PT_OFF_OWNER + PT_HT * 4;
constexpr u32 PT_OFF_AUX = PT_OFF_CNT + PT_TILE * 4;
constexpr u32 PT_OFF_LIST = PT_OFF_AUX + PT_TILE * 4;
constexpr u32 PT_OFF_LOWN = PT_OFF_LIST + PT_TILE * 2;
constexpr u32 PT_OFF_HIST = PT_OFF_LOWN + PT_TILE * 2;
constexpr u32 PT_MAX_PARTS = 4096;
constexpr u32 PT_LDS_FIXED = PT_OFF_HIST;  // 114688, then one word per partition

template <typename T>
__global__ __launch_bounds__(PT_BLOCK) void part_tile_kernel(
    TableDev t, const u64* __restrict__ keys, const T* __restrict__ grads, const u32* __restrict__ handles, u32 n,
    u32 P, u32 part_shift, uint4* __restrict__ stage, u32* __restrict__ starts, T* __restrict__ psum, u32 units) {
    extern __shared__ __align__(16) unsigned char pt_lds[];
    u64* lkey = reinterpret_cast<u64*>(pt_lds);
    u32* owner = reinterpret_cast<u32*>(pt_lds + PT_OFF_OWNER);
    u32* cnt = reinterpret_cast<u32*>(pt_lds + PT_OFF_CNT);
    u32* aux = reinterpret_cast<u32*>(pt_lds + PT_OFF_AUX);
    u16* list = reinterpret_cast<u16*>(pt_lds + PT_OFF_LIST);
    u16* lown = reinterpret_cast<u16*>(pt_lds + PT_OFF_LOWN);
    u32* hist = reinterpret_cast<u32*>(pt_lds + PT_OFF_HIST);
    __shared__ u64 sums[PT_BLOCK / 64];
    constexpr u32 N = sizeof(T) / 4;
    const u32 tid = threadIdx.x;
    const u32 tile = blockIdx.x;
    const u64 tb = (u64)tile * PT_TILE;

    u64 key[PT_ITEMS], hh[PT_ITEMS];
    u32 hdl[PT_ITEMS];
    bool valid[PT_ITEMS];
    u32 nbad = 0;
#pragma unroll
    for (u32 j = 0; j < PT_ITEMS; ++j) {  // no branch around a load: the four stay in flight together
        const u64 i = tb + j * PT_BLOCK + tid;
        key[j] = keys[i < n ? i : (u64)n - 1];
    }
#pragma unroll
    for (u32 j = 0; j < PT_ITEMS; ++j) {
        const u64 i = tb + j * PT_BLOCK + tid;
        hdl[j] = ROW_NONE;
        if (handles) hdl[j] = handles[i < n ? i : (u64)n - 1];  // (block-uniform branch)
    }
#pragma unroll
    for (u32 j = 0; j < PT_ITEMS; ++j) {
        const u32 q = j * PT_BLOCK + tid;
        const u64 i = tb + q;
        if (i >= n) key[j] = KEY_EMPTY;
        valid[j] = i < n && key[j] < KEY_DELETED;
        nbad += (i < n && !valid[j]) ? 1u : 0u;
        lkey[q] = key[j];
        cnt[q] = 0;
        hh[j] = hash64(key[j]);
    }
#pragma unroll
    for (u32 x = 0; x < PT_HT / PT_BLOCK; ++x) owner[x * PT_BLOCK + tid] = NONE32;
    for (u32 x = tid; x < P; x += PT_BLOCK) hist[x] = 0;
    if (nbad) atomicAdd(&t.counters[CNT_BADKEY], nbad);  // reserved keys are skipped (and rare)
    if (tile == 0 && tid == 0) t.counters[CNT_ANY_NEW] = 0u;
    __syncthreads();

    // the items of one key agree on a representative and number themselves
    u32 rep[PT_ITEMS], arr[PT_ITEMS];
#pragma unroll
    for (u32 j = 0; j < PT_ITEMS; ++j) {
        rep[j] = arr[j] = 0;
        if (valid[j]) dedupe_insert(key[j], j * PT_BLOCK + tid, hh[j], lkey, owner, cnt, PT_HT - 1, rep[j], arr[j]);
    }
    __syncthreads();

    // keys that repeat: a number each (in thread order) and a range of the item list
    u32 m[PT_ITEMS];
    bool isrep[PT_ITEMS], multi[PT_ITEMS];
    u32 my_multi = 0, my_len = 0;
#pragma unroll
    for (u32 j = 0; j < PT_ITEMS; ++j) {
        m[j] = valid[j] ? cnt[rep[j]] : 0u;
        isrep[j] = valid[j] && rep[j] == j * PT_BLOCK + tid;
        multi[j] = isrep[j] && m[j] >= 2;
        my_multi += multi[j] ? 1u : 0u;
        my_len += multi[j] ? m[j] : 0u;
    }
    u64 tot = 0;
    const u64 ex = block_scan_excl<PT_BLOCK>(((u64)my_len << 32) | my_multi, tid, sums, &tot);
    const u32 n_multi = (u32)tot, n_elems = (u32)(tot >> 32);
    u32* mrep = cnt + (PT_TILE - PT_MAX_MULTI);  // (the counts have been read: barriers of the scan since)
    {
        u32 mr = (u32)ex, lo = (u32)(ex >> 32);
#pragma unroll
        for (u32 j = 0; j < PT_ITEMS; ++j)
            if (multi[j]) {
                aux[j * PT_BLOCK + tid] = lo | (mr << 16);
                mrep[mr] = j * PT_BLOCK + tid;
                ++mr;
                lo += m[j];
            }
    }
    __syncthreads();
#pragma unroll
    for (u32 j = 0; j < PT_ITEMS; ++j)
        if (valid[j] && m[j] >= 2) {
            const u32 a = aux[rep[j]];
            list[(a & 0xFFFFu) + arr[j]] = (u16)(j * PT_BLOCK + tid);
            lown[(a & 0xFFFFu) + arr[j]] = (u16)(a >> 16);
        }

    // one entry per distinct key, grouped by partition in the tile's staging block
    u32 prank[PT_ITEMS], part[PT_ITEMS];
#pragma unroll
    for (u32 j = 0; j < PT_ITEMS; ++j) {
        part[j] = partition_of(t, hh[j], part_shift);
        prank[j] = isrep[j] ? atomicAdd(&hist[part[j]], 1u) : 0u;
    }
    __syncthreads();

    // Pre-summed rows of the keys that repeat, as many lists per round as the accumulators hold
    // (the room of the key array, the hash table and the first half of the counts, which nobody
    // reads any more). The rows of the first round are
    // requested now and added up after the staging block is written: their latency covers that.
    double* acc = reinterpret_cast<double*>(pt_lds);
    const u32 G = units;  // lanes per row (the host admits units <= PT_BLOCK)
    const u32 NG = PT_BLOCK / G;
    const u32 g = tid / G, c = tid - g * G;
    const bool on = g < NG;
    const u32 B = PT_ACC_DOUBLES / (units * N);  // lists per round, at least 1
    const T* tile_grads = grads + tb * units;
    constexpr u32 PF = 8;
    T pv[PF];
    u32 pl[PF];
    const u32 first_b1 = B < n_multi ? B : n_multi;
    const u32 first_hi = first_b1 < n_multi ? (aux[mrep[first_b1]] & 0xFFFFu) : n_elems;
    for (u32 x = tid; x < first_b1 * units * N; x += PT_BLOCK) acc[x] = 0.0;
    const u32 first_len = chunk_len(0u, first_hi, NG);
    const u32 my_first = g * first_len < first_hi ? g * first_len : first_hi;
    const u32 my_last = my_first + first_len < first_hi ? my_first + first_len : first_hi;
#pragma unroll
    for (u32 k = 0; k < PF; ++k) {
        const u32 e = my_first + k;
        const bool ok = on && e < my_last;
        pl[k] = ok ? (u32)lown[e] : NONE32;
        const u32 q = ok ? (u32)list[e] : 0u;  // (a lane without an element loads row 0 and drops it)
        pv[k] = tile_grads[(size_t)q * units + (on ? c : 0u)];
    }
    {
        // thread x owns PP consecutive partitions (P is a power of two, at least 64): where their
        // entries start in the staging block -- starts[tile][p], P + 1 words per tile, the last one
        // the tile's entry count
        const u32 PP = P > PT_BLOCK ? P / PT_BLOCK : 1u;
        u32 cc[PT_MAX_PARTS / PT_BLOCK];
        u32 local = 0;
#pragma unroll
        for (u32 x = 0; x < PT_MAX_PARTS / PT_BLOCK; ++x) {
            const u32 p = tid * PP + x;
            cc[x] = (x < PP && p < P) ? hist[p] : 0u;
            local += cc[x];
        }
        u64 all = 0;
        u32 run = (u32)block_scan_excl<PT_BLOCK>(local, tid, sums, &all);
        u32* my_starts = starts + (size_t)tile * (P + 1u);
        if (tid == 0) my_starts[P] = (u32)all;
#pragma unroll
        for (u32 x = 0; x < PT_MAX_PARTS / PT_BLOCK; ++x) {
            const u32 p = tid * PP + x;
            if (x < PP && p < P) {
                hist[p] = run;
                my_starts[p] = run;
                run += cc[x];
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (u32 j = 0; j < PT_ITEMS; ++j)
        if (isrep[j]) {
            const u64 pos = tb + hist[part[j]] + prank[j];
            const u32 ref = multi[j] ? (REF_PSUM | (tile * PT_MAX_MULTI + (aux[j * PT_BLOCK + tid] >> 16)))
                                     : (u32)(tb + j * PT_BLOCK + tid);
            stage[pos] = make_uint4((u32)key[j], (u32)(key[j] >> 32), ref, hdl[j]);
        }
    if (n_multi == 0) return;  // block-uniform

    for (u32 b0 = 0; b0 < n_multi; b0 += B) {
        const u32 b1 = b0 + B < n_multi ? b0 + B : n_multi;
        const u32 lo = aux[mrep[b0]] & 0xFFFFu;
        const u32 hi = b1 < n_multi ? (aux[mrep[b1]] & 0xFFFFu) : n_elems;
        auto row_of = [&](u32 e) { return tile_grads + (size_t)list[e] * units; };
        if (b0 == 0) {  // the accumulators are zero (barriers since) and the first rows are here
            if (on) {
                ListSum<T> ls;
                ls.begin(acc, 0u, units, c);
#pragma unroll
                for (u32 k = 0; k < PF; ++k)
                    if (pl[k] != NONE32) ls.take(pl[k], pv[k]);
                flat_sum_from<T>(row_of, lown, my_first + PF < my_last ? my_first + PF : my_last, my_last, c, ls);
                ls.flush();
            }
        } else {
            for (u32 x = tid; x < (b1 - b0) * units * N; x += PT_BLOCK) acc[x] = 0.0;
            __syncthreads();
            if (on) flat_sum<T>(row_of, lown, lo, hi, b0, acc, units, NG, g, c);
        }
        __syncthreads();
        if (on)
            for (u32 l = b0 + g; l < b1; l += NG)
                psum[((size_t)tile * PT_MAX_MULTI + l) * units + c] =
                    Acc<T>::load(acc + ((size_t)(l - b0) * units + c) * N);
        __syncthreads();
    }
}

// ---- 2. apply -------------------------------------------------------------------------------------
// LDS (dynamic, 72 KiB): entry keys | hash table (later the accumulators) | entry handles | aux |
// entry references (later the rows of the distinct keys) | references grouped by key | list numbers |
// distinct keys | keys with more than one entry.
constexpr u32 PA_OFF_OWNER = PA_CAP * 8;
constexpr u32 PA_OFF_HDL = PA_OFF_OWNER + PA_HT * 4;
constexpr u32 PA_OFF_AUX = PA_OFF_HDL + PA_CAP * 4;
constexpr u32 PA_OFF_LREF = PA_OFF_AUX + PA_CAP * 4;
constexpr u32 PA_OFF_LIST = PA_OFF_LREF + PA_CAP * 4;
constexpr u32 PA_OFF_LOWN = PA_OFF_LIST + PA_CAP * 4;
constexpr u32 PA_OFF_UREP = PA_OFF_LOWN + PA_CAP * 2;
constexpr u32 PA_OFF_MREP = PA_OFF_UREP + PA_CAP * 2;
constexpr u32 PA_OFF_SUMS = PA_OFF_MREP + PA_CAP * 2;          // partial sums of the block scans
constexpr u32 PA_OFF_MISC = PA_OFF_SUMS + (PA_BLOCK / 64) * 8;  // three counters
constexpr u32 PA_LDS = PA_OFF_MISC + 64;  // 75904

struct ApplyArgs {
    const uint4* stage;  // {key low, key high, reference, row handle}, a block of PT_TILE per tile
    const u32* starts;   // [tile][P + 1]: where each partition's entries start in the tile's block
    u32* pstart;         // out: entries in lower partitions (where the partition parks its new keys)
    u32 n_tiles, P, n_keys;
    u32 search_step;     // half the power of two that n_tiles rounds up to
    u32* new_slot;
    u32* new_count;
    u32 units;
    int insert;
    u32 cap;  // entries a pass holds: PA_CAP, or less when a test wants to see the passes
    int handles;  // the entries carry rows that an earlier pull reported
    int verify;   // ... which count only where row_keys agrees
    const u32* order;  // the work item of each workgroup (see rank_partitions), or null
    u32* psize;        // out: entries of each partition
    u32* resv;         // per partition, zero: where the workgroups that share a partition reserve room for new keys
};

// The optimizer step of the distinct keys of a pass: a key with one entry takes its gradient row, a
// key with several the sum that lies in the accumulators (lists below n_summed; the others are
// left to later rounds). Lane group g takes keys g, g + NG, ..., KS of them at a time, so that the
// loads of KS gradient rows and KS table rows are in flight together.
template <typename T, int KIND, u32 KS>
__device__ __forceinline__ void apply_keys(const TableDev& t, unsigned char* lds, const T* __restrict__ grads,
                                           const T* __restrict__ psum, T* __restrict__ ngrad, u32 s, u32 U, u32 units,
                                           u32 NG, u32 g, u32 c, const double* acc, u32 n_summed) {
    constexpr u32 N = sizeof(T) / 4;
    constexpr int STATES = states_of<KIND>();
    const u32* aux = reinterpret_cast<const u32*>(lds + PA_OFF_AUX);
    const u32* urow = reinterpret_cast<const u32*>(lds + PA_OFF_LREF);
    const u32* list = reinterpret_cast<const u32*>(lds + PA_OFF_LIST);
    const u16* urep = reinterpret_cast<const u16*>(lds + PA_OFF_UREP);
    T* rows = reinterpret_cast<T*>(t.rows);
    const u32 stride_units = t.stride_f / N;
    for (u32 u0 = g; u0 < U; u0 += KS * NG) {
        u32 rowk[KS], dst[KS];
        bool single[KS], isnew[KS];
        T gv[KS], wv[KS], av[STATES >= 1 ? KS : 1], bv[STATES >= 2 ? KS : 1];
#pragma unroll
        for (u32 k = 0; k < KS; ++k) {
            const u32 u = u0 + k * NG;
            single[k] = false;
            isnew[k] = false;
            rowk[k] = ROW_NONE;
            dst[k] = 0;
            gv[k] = vzero(T());
            u32 ref = 0;          // (a lane with nothing to fetch loads row 0 and drops it:
            bool summed = false;  // no branch around the loads, so that all of them are in flight)
            u32 mi = 0;
            if (u < U) {
                const u32 i = urep[u];
                const u32 av_ = aux[i];
                if (av_ & AUX_SINGLE) {
                    single[k] = true;
                    ref = list[av_ & 0xFFFFu];
                } else {
                    mi = (av_ >> 16) & AUX_MULTI_MASK;
                    summed = mi < n_summed;
                    single[k] = summed;
                }
                if (single[k]) {
                    isnew[k] = (av_ & AUX_NEW) != 0;
                    dst[k] = urow[u];
                    if (!isnew[k] && dst[k] < t.max_rows) rowk[k] = dst[k];
                }
            }
            gv[k] = ((ref & REF_PSUM) ? psum + (size_t)(ref & ~REF_PSUM) * units : grads + (size_t)ref * units)[c];
            if (summed) gv[k] = Acc<T>::load(acc + ((size_t)mi * units + c) * N);
        }
#pragma unroll
        for (u32 k = 0; k < KS; ++k) {
            const T* r = rows + (size_t)(rowk[k] != ROW_NONE ? rowk[k] : 0u) * stride_units + c;
            wv[k] = r[0];
            if constexpr (STATES >= 1) av[k] = r[units];
            if constexpr (STATES >= 2) bv[k] = r[2 * units];
        }
#pragma unroll
        for (u32 k = 0; k < KS; ++k) {
            if (!single[k]) continue;
            if (isnew[k]) {
                ngrad[(size_t)(s + dst[k]) * units + c] = gv[k];
            } else if (rowk[k] != ROW_NONE) {
                T a0 = vzero(T()), b0 = vzero(T());
                if constexpr (STATES >= 1) a0 = av[k];
                if constexpr (STATES >= 2) b0 = bv[k];
                float* gp = reinterpret_cast<float*>(&gv[k]);
                float* wp = reinterpret_cast<float*>(&wv[k]);
                float* ap = reinterpret_cast<float*>(&a0);
                float* bp = reinterpret_cast<float*>(&b0);
#pragma unroll
                for (u32 e = 0; e < N; ++e) opt_step<KIND>(t.opt, gp[e], wp[e], ap[e], bp[e]);
                T* r = rows + (size_t)rowk[k] * stride_units + c;
                if (t.dirty && c == 0) t.dirty[rowk[k]] = 1;
                r[0] = wv[k];
                if constexpr (STATES >= 1) r[units] = a0;
                if constexpr (STATES >= 2) r[2 * units] = b0;
            }
        }
    }
}

// Everything a pass does with the `count` entries that lie in lkey / lref.
template <typename T>
__device__ __forceinline__ void apply_pass(const TableDev& t, unsigned char* lds, u64* sums, u32* s_nnew,
                                           const T* __restrict__ grads, const T* __restrict__ psum,
                                           T* __restrict__ ngrad, const ApplyArgs& a, u32 s, u32 count) {
    constexpr u32 N = sizeof(T) / 4;
    u64* lkey = reinterpret_cast<u64*>(lds);
    u32* owner = reinterpret_cast<u32*>(lds + PA_OFF_OWNER);
    const u32* lhdl = reinterpret_cast<const u32*>(lds + PA_OFF_HDL);
    u32* aux = reinterpret_cast<u32*>(lds + PA_OFF_AUX);
    u32* lref = reinterpret_cast<u32*>(lds + PA_OFF_LREF);
    u32* list = reinterpret_cast<u32*>(lds + PA_OFF_LIST);
    u16* lown = reinterpret_cast<u16*>(lds + PA_OFF_LOWN);
    u16* urep = reinterpret_cast<u16*>(lds + PA_OFF_UREP);
    u16* mrep = reinterpret_cast<u16*>(lds + PA_OFF_MREP);
    const u32 tid = threadIdx.x, lane = tid & 63u;
    const u32 units = a.units;

    u32& s_nwalk = reinterpret_cast<u32*>(lds + PA_OFF_MISC)[5];  // keys that take the walk
    if (tid == 0) s_nwalk = 0;
#pragma unroll
    for (u32 x = 0; x < PA_HT / PA_BLOCK; ++x) owner[x * PA_BLOCK + tid] = NONE32;
    __syncthreads();

    u32 rep[PA_ITEMS], arr[PA_ITEMS], hslot[PA_ITEMS];
    bool valid[PA_ITEMS];
#pragma unroll
    for (u32 j = 0; j < PA_ITEMS; ++j) {
        const u32 i = j * PA_BLOCK + tid;
        valid[j] = i < count;
        rep[j] = arr[j] = hslot[j] = 0;
        if (valid[j]) {
            const u64 key = lkey[i];
            dedupe_insert_packed(key, i, hash64(key), lkey, owner, PA_HT - 1, rep[j], arr[j], hslot[j]);
        }
    }
    __syncthreads();

    // distinct keys numbered; the references of the keys with several entries come first in the list
    u32 m[PA_ITEMS];
    bool isrep[PA_ITEMS];
    u32 my_u = 0, my_multi = 0, my_len = 0;
#pragma unroll
    for (u32 j = 0; j < PA_ITEMS; ++j) {
        m[j] = valid[j] ? owner[hslot[j]] >> 16 : 0u;
        isrep[j] = valid[j] && rep[j] == j * PA_BLOCK + tid;
        my_u += isrep[j] ? 1u : 0u;
        my_multi += (isrep[j] && m[j] >= 2) ? 1u : 0u;
        my_len += (isrep[j] && m[j] >= 2) ? m[j] : 0u;
    }
    u64 tot = 0;
    const u64 ex = block_scan_excl<PA_BLOCK>((u64)my_u | ((u64)my_multi << 16) | ((u64)my_len << 32), tid, sums, &tot);
    const u32 U = (u32)(tot & 0xFFFFu), n_multi = (u32)((tot >> 16) & 0xFFFFu), n_elems = (u32)(tot >> 32);
    {
        u32 ur = (u32)(ex & 0xFFFFu), mr = (u32)((ex >> 16) & 0xFFFFu), lo = (u32)(ex >> 32);
#pragma unroll
        for (u32 j = 0; j < PA_ITEMS; ++j)
            if (isrep[j]) {
                const u32 i = j * PA_BLOCK + tid;
                urep[ur] = (u16)i;
                if (m[j] >= 2) {
                    aux[i] = lo | (mr << 16);
                    mrep[mr] = (u16)ur;  // the key's number among the distinct keys
                    ++mr;
                    lo += m[j];
                } else {
                    aux[i] = (n_elems + (ur - mr)) | AUX_SINGLE;  // single entries follow the lists
                }
                ++ur;
            }
    }
    __syncthreads();
#pragma unroll
    for (u32 j = 0; j < PA_ITEMS; ++j)
        if (valid[j]) {
            const u32 av = aux[rep[j]];
            const u32 pos = (av & 0xFFFFu) + arr[j];
            list[pos] = lref[j * PA_BLOCK + tid];
            lown[pos] = (u16)((av >> 16) & AUX_MULTI_MASK);
        }
    // the hash table is done with: its room becomes the accumulators of the keys with several entries,
    // as many lists as it holds (normally all of them)
    double* acc = reinterpret_cast<double*>(owner);
    const u32 B = PA_ACC_DOUBLES / (units * N);
    const u32 first_b1 = B < n_multi ? B : n_multi;
    for (u32 x = tid; x < first_b1 * units * N; x += PA_BLOCK) acc[x] = 0.0;
    __syncthreads();
    const u32 G = units;  // the host admits units <= PA_BLOCK
    const u32 NG = PA_BLOCK / G;
    const u32 g = tid / G, c = tid - g * G;
    const bool on = g < NG;
    auto src = [&](u32 ref) -> const T* {
        return (ref & REF_PSUM) ? psum + (size_t)(ref & ~REF_PSUM) * units : grads + (size_t)ref * units;
    };
    bool sums_due = n_multi != 0;  // block-uniform
    const u32 first_hi = first_b1 < n_multi ? (aux[urep[mrep[first_b1]]] & 0xFFFFu) : n_elems;

    // One probe per distinct key, four lanes each. A lane group looks at the home buckets of
    // several keys at once (all the loads in flight together); a key that is not in its home
    // bucket -- or must claim a slot -- then takes the ordinary walk. A key whose entries carry the
    // row an earlier pull found is not looked up at all (with `verify`: once row_keys has
    // confirmed it, a load that goes out with the bucket loads of the other keys).
    u32* urow = lref;
    const u32 grp = lane >> 2, sub = lane & 3u;
    constexpr u32 KP = 4, QUADS = PA_BLOCK / 4;
    const u32 rows_now = t.counters[CNT_ROWS];  // (this launch hands out no rows)
    for (u32 u0 = 0; u0 < U; u0 += QUADS * KP) {
        u32 uu[KP], ii[KP], hd[KP];
        u64 kk[KP], vk[KP] = {};
        bool act[KP], byh[KP];
        uint4 sv[KP] = {};
        bool any_lookup = false;
#pragma unroll
        for (u32 k = 0; k < KP; ++k) {
            uu[k] = u0 + k * QUADS + (tid >> 2);
            act[k] = uu[k] < U;
            ii[k] = act[k] ? urep[uu[k]] : 0u;
            kk[k] = act[k] ? lkey[ii[k]] : KEY_EMPTY;
            hd[k] = lhdl[ii[k]];
            byh[k] = act[k] && a.handles && hd[k] < rows_now;
            any_lookup |= act[k] && !byh[k];
        }
        const bool wave_looks = __ballot(any_lookup) != 0;  // wavefront-uniform
        if (wave_looks) {
#pragma unroll
            for (u32 k = 0; k < KP; ++k)  // (a lane group with a handle reads bucket 0 and drops it)
                sv[k] = t.slots[(u64)(byh[k] ? 0u : ((u32)hash64(kk[k]) & t.bucket_mask)) * 4 + sub];
        }
        if (a.verify) {
#pragma unroll
            for (u32 k = 0; k < KP; ++k) vk[k] = t.row_keys[byh[k] ? hd[k] : 0u];
        }
        if (sums_due) {  // while the loads are on their way: the sums of the keys with several entries
            if (on) flat_sum<T>([&](u32 e) { return src(list[e]); }, lown, 0u, first_hi, 0u, acc, units, NG, g, c);
            sums_due = false;
        }
        bool late[KP];  // a handle that row_keys does not confirm: looked up after all
#pragma unroll
        for (u32 k = 0; k < KP; ++k) {
            late[k] = false;
            if (a.verify && byh[k] && vk[k] != kk[k]) {
                byh[k] = false;
                late[k] = true;
            }
            if (byh[k] && sub == 0) urow[uu[k]] = hd[k];
        }
        if (!wave_looks && !(a.verify && __ballot(late[0] || late[1] || late[2] || late[3]))) continue;
#pragma unroll
        for (u32 k = 0; k < KP; ++k) {
            const bool look = act[k] && !byh[k];
            const u64 skey = ((u64)sv[k].y << 32) | sv[k].x;
            const bool home = wave_looks && look && !late[k];  // sv[k] is the key's home bucket
            const bool match = home && skey == kk[k];
            const bool empty = home && skey == KEY_EMPTY;
            const u32 m4 = (u32)(__ballot(match) >> (grp * 4)) & 0xFu;
            const u32 e4 = (u32)(__ballot(empty) >> (grp * 4)) & 0xFu;
            const u32 srcl = grp * 4 + (m4 ? (u32)__ffs((int)m4) - 1u : 0u);
            const u32 hrow = __shfl(wave_looks ? sv[k].z : 0u, (int)srcl);
            // found at home: done. Absent for sure (an empty slot at home) and nothing to insert: done.
            // Everything else -- a key that is not in its home bucket, a key to insert -- takes the
            // ordinary walk, and not here: such keys are few per wavefront, and a walk (or a claim,
            // a round trip of an atomic) at this point would hold up sixteen keys for one. They are
            // marked, and collected below.
            const bool slow = look && (!home || (!m4 && (a.insert || !e4)));
            if (look && sub == 0) urow[uu[k]] = slow ? ROW_WALK : (m4 && hrow < t.max_rows) ? hrow : ROW_NONE;
        }
    }
    __syncthreads();
    // The marked keys, packed (the handles have been read: the queue takes their room), one per
    // lane group and all lane groups at once.
    {
        u16* queue = reinterpret_cast<u16*>(lds + PA_OFF_HDL);
        for (u32 u = tid; u < U; u += PA_BLOCK)
            if (urow[u] == ROW_WALK) queue[atomicAdd(&s_nwalk, 1u)] = (u16)u;
        __syncthreads();
        const u32 n_walk = s_nwalk;  // block-uniform
        for (u32 q0 = 0; q0 < n_walk; q0 += QUADS) {
            const u32 q = q0 + (tid >> 2);
            const bool on_q = q < n_walk;
            const u32 u = on_q ? (u32)queue[q] : 0u;
            const u32 i = urep[u];
            const u64 key = on_q ? lkey[i] : KEY_EMPTY;
            u32 row = ROW_NONE, slot = SLOT_NONE;
            bool won = false;
            if (a.insert) {
                const Located l = find_or_claim(t, key, on_q, grp, sub, true);
                row = l.row;
                slot = l.slot;
                won = l.won;
            } else {
                const Found f = probe_find(t, key, on_q, grp, sub);
                row = f.row;
            }
            if (on_q && sub == 0) {
                if (won) {
                    const u32 kn = atomicAdd(s_nnew, 1u);
                    a.new_slot[s + kn] = slot;
                    urow[u] = kn;
                    aux[i] |= AUX_NEW;
                } else {
                    urow[u] = row < t.max_rows ? row : ROW_NONE;
                }
            }
        }
        if (n_walk) __syncthreads();
    }

    auto apply = [&](u32 u, u32 i, T gv) {
        if (aux[i] & AUX_NEW) {
            ngrad[(size_t)(s + urow[u]) * units + c] = gv;
        } else {
            const u32 row = urow[u];
            if (row != ROW_NONE) finalize<T>(t, row, c, units, gv);
        }
    };
    // one sweep over the distinct keys: step and store
    if (on) {
        switch (t.opt.kind) {
            case 0: apply_keys<T, 0, 4>(t, lds, grads, psum, ngrad, s, U, units, NG, g, c, acc, first_b1); break;
            case 1: apply_keys<T, 1, 4>(t, lds, grads, psum, ngrad, s, U, units, NG, g, c, acc, first_b1); break;
            case 2: apply_keys<T, 2, 2>(t, lds, grads, psum, ngrad, s, U, units, NG, g, c, acc, first_b1); break;
            case 3: apply_keys<T, 3, 2>(t, lds, grads, psum, ngrad, s, U, units, NG, g, c, acc, first_b1); break;
            default: apply_keys<T, 4, 2>(t, lds, grads, psum, ngrad, s, U, units, NG, g, c, acc, first_b1); break;
        }
    }
    // more lists than the accumulators hold (rows of several KiB): further rounds
    for (u32 b0 = first_b1; b0 < n_multi; b0 += B) {
        const u32 b1 = b0 + B < n_multi ? b0 + B : n_multi;
        const u32 lo = aux[urep[mrep[b0]]] & 0xFFFFu;
        const u32 hi = b1 < n_multi ? (aux[urep[mrep[b1]]] & 0xFFFFu) : n_elems;
        __syncthreads();
        for (u32 x = tid; x < (b1 - b0) * units * N; x += PA_BLOCK) acc[x] = 0.0;
        __syncthreads();
        if (on) flat_sum<T>([&](u32 e) { return src(list[e]); }, lown, lo, hi, b0, acc, units, NG, g, c);
        __syncthreads();
        if (on)
            for (u32 l = b0 + g; l < b1; l += NG) {
                const u32 u = mrep[l];
                apply(u, urep[u], Acc<T>::load(acc + ((size_t)(l - b0) * units + c) * N));
            }
    }
}

// The partition's segments in the staging blocks: tile x holds entries [ta[x], ta[x] + count) of its
// block, and they are entries toff[x] .. of the partition (toff is filled for all PA_TILES_MAX
// numbers, with the partition's entry count beyond the last tile). A thread takes two tiles; the
// loads are issued before anything waits. Returns {entries of the partition, entries in lower
// partitions}. All threads call it.
constexpr u32 PA_TILES_MAX = 2 * PA_BLOCK;
constexpr u32 ORDER_TAG = PART_ORDER_TAG;  // where the order names its plan: {partitions, bucket mask}
static_assert(PT_MAX_PARTS == PART_MAX_PARTS, "the order's layout follows the largest cut");
constexpr u32 PA_STACK = 72;  // classes that can wait at once: one per bit of the second hash, and a few
static_assert(PA_CAP + PA_STACK * 12 <= PA_CAP * 2, "the stack fits the upper half of mrep");

// The second hash, by which a crowded partition is taken in passes: one-to-one like hash64, and
// unrelated to the bits of hash64 that choose partition and bucket.
__device__ __forceinline__ u64 class_hash(u64 key) { return hash64(hash64(key) ^ 0x9E3779B97F4A7C15ull); }
static_assert(PART_MAX_KEYS / PT_TILE <= PA_TILES_MAX, "two tiles per thread cover the largest batch");
static_assert(2 * PA_TILES_MAX <= PA_CAP, "the offsets fit the room of the reference list");

__device__ __forceinline__ u64 tile_segments(const ApplyArgs& a, u32 p, u32 tid, u64* sums, u32* toff, u32* ta) {
    const u32 x0 = 2u * tid, x1 = x0 + 1u;
    const size_t stride = (size_t)a.P + 1u;
    const u32* c0 = a.starts + (size_t)(x0 < a.n_tiles ? x0 : 0u) * stride + p;
    const u32* c1 = a.starts + (size_t)(x1 < a.n_tiles ? x1 : 0u) * stride + p;
    u32 a0 = c0[0], b0 = c0[1], a1 = c1[0], b1 = c1[1];
    if (x0 >= a.n_tiles) a0 = b0 = 0u;
    if (x1 >= a.n_tiles) a1 = b1 = 0u;
    const u32 n0 = b0 - a0, n1 = b1 - a1;
    u64 tot = 0;
    const u64 ex = block_scan_excl<PA_BLOCK>((u64)(n0 + n1) | ((u64)(a0 + a1) << 32), tid, sums, &tot);
    toff[x0] = (u32)ex;
    toff[x1] = (u32)ex + n0;
    ta[x0] = a0;
    ta[x1] = a1;
    return tot;
}

// entry i of the partition (tile_segments() has run, a barrier since)
__device__ __forceinline__ uint4 partition_entry(const ApplyArgs& a, const u32* toff, const u32* ta, u32 i) {
    u32 x = 0;
    for (u32 step = a.search_step; step; step >>= 1)
        if (toff[x + step] <= i) x += step;  // the last tile that starts at or before entry i
    return a.stage[(size_t)x * PT_TILE + ta[x] + (i - toff[x])];
}

// A partition with more entries than a pass holds (several keys that are met in most tiles share
// it) is taken in passes by hash class, a class being the keys that agree in the low bits of a
// second hash: first two classes; one that still holds too many is split in two by the next bit,
// as often as it takes -- the second hash is one-to-one, so two keys part company at some bit, and
// one key alone has at most an entry per tile, which a pass holds. (Only a pass capacity below the
// number of tiles, which a test may set, can leave a class of one key too large; that is
// reported.) The classes still to do wait on a stack in the upper half of the room of `mrep`,
// which no pass touches (it numbers keys with several entries: at most half a pass).
template <typename T>
__device__ __forceinline__ void apply_crowded(const TableDev& t, unsigned char* pa_lds, const T* __restrict__ grads,
                                              const T* __restrict__ psum, T* __restrict__ ngrad, const ApplyArgs& a,
                                              u32 p, u32 s, u32 np, u32 lg0, u32 cls0, u32 unit) {
    u64* sums = reinterpret_cast<u64*>(pa_lds + PA_OFF_SUMS);
    u32* misc = reinterpret_cast<u32*>(pa_lds + PA_OFF_MISC);
    u32& s_sel = misc[1];
    u32& s_sp = misc[2];
    u64* lkey = reinterpret_cast<u64*>(pa_lds);
    u32* lref = reinterpret_cast<u32*>(pa_lds + PA_OFF_LREF);
    u32* lhdl = reinterpret_cast<u32*>(pa_lds + PA_OFF_HDL);
    u32* toff = reinterpret_cast<u32*>(pa_lds + PA_OFF_LIST);
    u32* ta = toff + PA_TILES_MAX;
    u64* stk_cls = reinterpret_cast<u64*>(pa_lds + PA_OFF_MREP + PA_CAP);
    u32* stk_lg = reinterpret_cast<u32*>(stk_cls + PA_STACK);
    const u32 tid = threadIdx.x;
    if (tid == 0) {
        if (lg0) {  // this workgroup's share of a partition that several take: one class
            stk_cls[0] = cls0;
            stk_lg[0] = lg0;
            s_sp = 1;
        } else {
            stk_cls[0] = 0;
            stk_cls[1] = 1;
            stk_lg[0] = stk_lg[1] = 1;
            s_sp = 2;
        }
    }
    // Workgroups that share a partition share its room for new keys: each reserves as much as its
    // class has entries (known after its first sweep) and parks its new keys there.
    bool reserve = lg0 != 0 && a.insert;  // block-uniform
    __syncthreads();
    while (s_sp) {  // block-uniform: read between barriers
        const u32 lg = stk_lg[s_sp - 1];
        const u64 cls = stk_cls[s_sp - 1];
        __syncthreads();
        if (tid == 0) {
            s_sp -= 1;
            s_sel = 0;
        }
        __syncthreads();
        const u64 mask = lg >= 64u ? ~0ull : (1ull << lg) - 1ull;
        tile_segments(a, p, tid, sums, toff, ta);  // (a pass overwrites them)
        __syncthreads();
        for (u32 i = tid; i < np; i += PA_BLOCK) {
            const uint4 e = partition_entry(a, toff, ta, i);
            const u64 key = ((u64)e.y << 32) | e.x;
            if ((class_hash(key) & mask) == cls) {
                const u32 pos = atomicAdd(&s_sel, 1u);
                if (pos < a.cap) {
                    lkey[pos] = key;
                    lref[pos] = e.z;
                    lhdl[pos] = e.w;
                }
            }
        }
        __syncthreads();
        const u32 sel = s_sel;
        if (reserve) {
            if (tid == 0) {
                misc[4] = atomicAdd(&a.resv[p], sel);
                a.pstart[unit] = s + misc[4];
            }
            __syncthreads();
            s += misc[4];
            reserve = false;
        }
        if (sel > a.cap) {
            if (lg >= 64u) {  // one key with more entries than a pass holds: reported, never silent
                if (tid == 0) t.counters[CNT_PART_ERR] = 1u;
            } else if (tid == 0) {  // (a pop and two pushes per level: never more than 65 waiting)
                stk_cls[s_sp] = cls;
                stk_lg[s_sp] = lg + 1u;
                stk_cls[s_sp + 1] = cls | (1ull << lg);
                stk_lg[s_sp + 1] = lg + 1u;
                s_sp += 2;
            }
        } else if (sel) {
            apply_pass<T>(t, pa_lds, sums, misc, grads, psum, ngrad, a, s, sel);
        }
        __syncthreads();
    }
}

template <typename T>
__global__ __launch_bounds__(PA_BLOCK, 4) void part_apply_kernel(TableDev t, const T* __restrict__ grads,
                                                               const T* __restrict__ psum, T* __restrict__ ngrad,
                                                               ApplyArgs a) {
    extern __shared__ __align__(16) unsigned char pa_lds[];
    u64* sums = reinterpret_cast<u64*>(pa_lds + PA_OFF_SUMS);
    u32& s_nnew = *reinterpret_cast<u32*>(pa_lds + PA_OFF_MISC);
    u64* lkey = reinterpret_cast<u64*>(pa_lds);
    u32* lref = reinterpret_cast<u32*>(pa_lds + PA_OFF_LREF);
    u32* lhdl = reinterpret_cast<u32*>(pa_lds + PA_OFF_HDL);
    u32* toff = reinterpret_cast<u32*>(pa_lds + PA_OFF_LIST);  // (the reference list is written later)
    u32* ta = toff + PA_TILES_MAX;
    const u32 tid = threadIdx.x;
    // Workgroups are dealt to the eight XCDs in turn: each XCD takes a run of consecutive partitions,
    // whose start words and staging segments share cache lines, into its own L2. With an order (the
    // partitions of each run ranked by the entries the last push found in them) the fullest go
    // first: a kernel of several rounds of workgroups ends when its last workgroup does, and a
    // crowded partition that starts in the last round would be that one.
    // A work item names a partition and, for one that the last push found crowded, one of the
    // 2, 4 or 8 classes of its keys (by the low bits of the second hash): that many workgroups
    // share it from the start instead of one taking its passes one after the other.
    // The order names the plan it was made for in the two words behind its slots: one left by a
    // push with another plan (a launch recorded earlier and replayed, say) is not followed.
    const u32 unit = blockIdx.x;
    const bool ordered = a.order && a.order[ORDER_TAG] == a.P && a.order[ORDER_TAG + 1] == t.bucket_mask;
    const u32 item = ordered ? a.order[unit] : unit < a.P ? (unit & 7u) * (a.P >> 3) + (unit >> 3) : NONE32;
    if (item == NONE32) {  // (block-uniform) a spare slot of the order
        if (tid == 0) a.new_count[unit] = 0;
        return;
    }
    const u32 p = item & 0xFFFFu, lg0 = (item >> 16) & 3u, cls0 = item >> 20;
    const u64 seg = tile_segments(a, p, tid, sums, toff, ta);
    const u32 np = (u32)seg, s = (u32)(seg >> 32);
    // the row count as it is when this operation begins (this launch hands out no rows)
    if (p == 0 && tid == 0) t.counters[CNT_ENTRY] = t.counters[CNT_ROWS];
    if (tid == 0) {
        s_nnew = 0;
        a.pstart[unit] = s;
        a.psize[p] = np;
        // the last partition's block knows how many entries the tiles left in all: a hint for the
        // partition size of the next push (read by the host when it plans that push)
        if (p + 1 == a.P)
            __hip_atomic_store(t.part_stat, ((unsigned long long)a.n_keys << 32) | (unsigned long long)(s + np),
                               __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_SYSTEM);
    }
    if (np == 0) {
        if (tid == 0) a.new_count[unit] = 0;
        return;
    }
    __syncthreads();
    if (__builtin_expect(np <= a.cap && lg0 == 0, 1)) {
        uint4 e[PA_ITEMS];
#pragma unroll
        for (u32 j = 0; j < PA_ITEMS; ++j) {
            const u32 i = j * PA_BLOCK + tid;
            e[j] = partition_entry(a, toff, ta, i < np ? i : 0u);
        }
#pragma unroll
        for (u32 j = 0; j < PA_ITEMS; ++j) {
            const u32 i = j * PA_BLOCK + tid;
            if (i < np) {
                lkey[i] = ((u64)e[j].y << 32) | e[j].x;
                lref[i] = e[j].z;
                lhdl[i] = e[j].w;
            }
        }
        __syncthreads();
        apply_pass<T>(t, pa_lds, sums, &s_nnew, grads, psum, ngrad, a, s, np);
    } else {
        apply_crowded<T>(t, pa_lds, grads, psum, ngrad, a, p, s, np, lg0, cls0, unit);
    }
    __syncthreads();
    if (tid == 0) {
        a.new_count[unit] = s_nnew;
        if (s_nnew) t.counters[CNT_ANY_NEW] = 1u;  // (every writer writes the same value)
    }
}

// ---- 3. insert ------------------------------------------------------------------------------------
constexpr u32 PI_BLOCK = 256;

// The work items for the apply kernel of the next push with this plan. Run g (P / 8 consecutive
// partitions, at most 512) gets P / 8 + P / 64 slots; workgroup x of that kernel is on XCD x & 7
// and takes slot x >> 3 of run x & 7. The partitions of the run are ranked by the entries this
// push found in them, fullest first (ties by number). Those that were crowded, or nearly (a pass
// holds PA_CAP entries), come first and get 2, 4 or 8 slots each while spare slots last: item =
// partition | log2(slots) << 16 | class << 20, each workgroup taking the keys of one class. The
// others follow with one slot each in their natural order -- neighbours share cache lines of start
// words and staging blocks, and run at about the same time that way -- and what is left of the
// spare slots says so (NONE32). Every partition is covered whatever the sizes are. The
// reservation words of the run are cleared for the next push.
constexpr u32 PART_SPLIT_ABOVE = PA_CAP - PA_CAP / 7;  // 1756 entries: crowded next time, for all we know
constexpr u32 PART_SHARE = 1300;                        // entries a workgroup of a shared partition should get

__host__ __device__ inline u32 part_units(u32 P, bool ordered) { return ordered ? P + P / 8 : P; }

__device__ __forceinline__ void rank_partitions(const u32* __restrict__ psize, u32* __restrict__ order,
                                                u32* __restrict__ resv, u32 P, u32 bucket_mask, u32 g, u32 tid) {
    __shared__ u32 sz[PT_MAX_PARTS / 8];
    __shared__ u16 sorted[PT_MAX_PARTS / 8], rank_of[PT_MAX_PARTS / 8];
    __shared__ u32 s_head, s_items;
    const u32 m = P >> 3, slots = m + (m >> 3);
    for (u32 i = tid; i < m; i += PI_BLOCK) {
        sz[i] = psize[g * m + i];
        resv[g * m + i] = 0;
    }
    if (g == 0 && tid == 0) {
        order[ORDER_TAG] = P;
        order[ORDER_TAG + 1] = bucket_mask;
    }
    __syncthreads();
    for (u32 i = tid; i < m; i += PI_BLOCK) {
        const u32 mine = sz[i];
        u32 rank = 0;
        for (u32 j = 0; j < m; ++j) {
            const u32 o = sz[j];
            rank += (o > mine || (o == mine && j < i)) ? 1u : 0u;
        }
        sorted[rank] = (u16)i;
        rank_of[i] = (u16)rank;
    }
    __syncthreads();
    if (tid == 0) {  // the partitions that get more than one slot are the first of the ranking
        u32 spare = m >> 3, pos = 0, r = 0;
        for (; r < m && spare; ++r) {
            const u32 i = sorted[r], size = sz[i];
            if (size <= PART_SPLIT_ABOVE) break;
            u32 lg = 1;
            while ((size >> lg) > PART_SHARE && lg < 3u) ++lg;
            while (lg && (1u << lg) - 1u > spare) --lg;
            if (lg == 0) break;
            spare -= (1u << lg) - 1u;
            for (u32 c = 0; c < (1u << lg); ++c) order[(pos++ << 3) | g] = (g * m + i) | (lg << 16) | (c << 20);
        }
        s_head = r;
        s_items = pos;
    }
    __syncthreads();
    const u32 head = s_head, items = s_items;
    for (u32 i = tid; i < m; i += PI_BLOCK) {
        if (rank_of[i] < head) continue;  // placed above
        u32 before = 0;                   // partitions below i that were
        for (u32 k = 0; k < head; ++k) before += sorted[k] < i ? 1u : 0u;
        order[((items + i - before) << 3) | g] = g * m + i;
    }
    for (u32 x = items + (m - head) + tid; x < slots; x += PI_BLOCK) order[(x << 3) | g] = NONE32;
}

template <typename T>
__global__ __launch_bounds__(PI_BLOCK) void part_insert_kernel(TableDev t, const u32* __restrict__ new_slot,
                                                                const T* __restrict__ ngrad,
                                                                const u32* __restrict__ new_count,
                                                                const u32* __restrict__ pstart, u32 P, u32 units,
                                                                const u32* __restrict__ psize, u32* __restrict__ order,
                                                                u32* __restrict__ resv, u32 n_parts, u32 n_rankers) {
    // P: workgroups the apply kernel had (one per partition, or the slots of its order); each left
    // its new keys parked at pstart[its number], new_count of them. n_parts: partitions.
    constexpr u32 N = sizeof(T) / 4;
    __shared__ u32 red[PI_BLOCK / 64];
    const u32 tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    // eight more workgroups when an order is wanted, one per run of n_parts / 8 partitions: the first
    // of the grid, because theirs is the longest job of the launch
    if (blockIdx.x < n_rankers) {
        rank_partitions(psize, order, resv, n_parts, t.bucket_mask, blockIdx.x, tid);
        return;
    }
    const u32 p = blockIdx.x - n_rankers;
    if (!t.counters[CNT_ANY_NEW]) {  // block-uniform: the batch inserted nothing
        if (p == 0 && tid == 0) publish_rows(t, t.counters[CNT_ENTRY]);
        return;
    }
    const u32 mine = new_count[p];
    if (mine == 0 && p != 0) return;  // block-uniform
    const u32 upto = p == 0 ? P : p;
    u32 part = 0;
    for (u32 x = tid; x < upto; x += PI_BLOCK) part += new_count[x];
    for (u32 off = 32; off >= 1; off >>= 1) part += __shfl_down(part, off);
    if (lane == 0) red[w] = part;
    __syncthreads();
    u32 sum = 0;
    for (u32 x = 0; x < PI_BLOCK / 64; ++x) sum += red[x];
    const u32 entry = t.counters[CNT_ENTRY];
    if (p == 0) {
        if (tid == 0) {
            t.counters[CNT_ROWS] = entry + sum;
            if (entry + sum > t.max_rows) t.counters[CNT_OVERFLOW] = 1u;
            publish_rows(t, entry + sum);
        }
        if (mine == 0) return;
        sum = 0;
    }
    const u32 first_row = entry + sum;
    const u32 s = pstart[p];
    const u32 G = units < PI_BLOCK ? units : PI_BLOCK;
    const u32 NG = PI_BLOCK / G;
    const u32 g = tid / G, c0 = tid - g * G;
    if (g >= NG) return;
    const u32 dim = t.dim;
    for (u32 k = g; k < mine; k += NG) {
        const u32 slot = new_slot[s + k];
        const u32 row = first_row + k;
        if (row >= t.max_rows) continue;  // does not fit (the host rules this out before it takes this path)
        const uint4 sv = t.slots[slot];
        const u64 key = ((u64)sv.y << 32) | sv.x;
        if (c0 == 0) {
            reinterpret_cast<u32*>(&t.slots[slot])[2] = row;
            t.row_keys[row] = key;
            if (t.dirty) t.dirty[row] = 1;
        }
        T* r = reinterpret_cast<T*>(t.rows + (size_t)row * t.stride_f);
        for (u32 c = c0; c < units; c += G) {
            T gv = ngrad[(size_t)(s + k) * units + c];
            T wv, av = vzero(T()), bv = vzero(T());
            float* gp = reinterpret_cast<float*>(&gv);
            float* wp = reinterpret_cast<float*>(&wv);
            float* ap = reinterpret_cast<float*>(&av);
            float* bp = reinterpret_cast<float*>(&bv);
#pragma unroll
            for (u32 x = 0; x < N; ++x) {
                wp[x] = init_float(t, key, c * N + x);
                ap[x] = init_float(t, key, dim + c * N + x);
                bp[x] = init_float(t, key, 2 * dim + c * N + x);
            }
            opt_step_n<(int)N>(t.opt, gp, wp, ap, bp);
            r[c] = wv;
            if (t.opt.states >= 1) r[units + c] = av;
            if (t.opt.states >= 2) r[2 * units + c] = bv;
        }
    }
}

inline bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }

}  // namespace

// ---- host side --------------------------------------------------------------------------------
namespace {
u32 g_part_cap = PA_CAP;
size_t g_part_min_keys = PART_MIN_KEYS;
}
void part_set_pass_capacity(uint32_t entries) { g_part_cap = entries == 0 || entries > PA_CAP ? PA_CAP : entries; }
void part_set_min_keys(size_t keys) { g_part_min_keys = keys == 0 ? PART_MIN_KEYS : keys; }

bool part_plan(const TableDev& t, size_t n, double entries_per_key, PartPlan* plan) {
    if (n < g_part_min_keys || n > PART_MAX_KEYS) return false;
    const u32 vec = (t.dim % 4 == 0) ? 4u : 1u;
    if (t.dim / vec > PA_BLOCK) return false;  // a lane per 4 or 16 bytes of a row
    u32 bucket_bits = 0;
    while ((1ull << bucket_bits) <= t.bucket_mask) ++bucket_bits;
    // A workgroup of the apply kernel is a chain of dependent round trips whatever it holds, so a
    // partition should fill a pass (PA_CAP entries) as far as it safely can: about PART_TARGET
    // entries on average (half that for long rows), which leaves room for the spread between partitions and for the entries
    // of a key that is met in every tile. At least 64 partitions, at most 4096.
    if (!(entries_per_key > 0.0 && entries_per_key <= 1.0)) entries_per_key = 1.0;
    const double entries = entries_per_key * (double)n;
    u32 lp = 6;
    const double target = t.dim <= 32 ? PART_TARGET : PART_TARGET_LONG_ROWS;
    while ((double)(1ull << lp) * target < entries && lp < 12) ++lp;
    if (lp > bucket_bits) return false;  // a tiny table under a large batch: the sort path serves it
    plan->n = (u32)n;
    plan->n_tiles = (u32)((n + PT_TILE - 1) / PT_TILE);
    plan->P = 1u << lp;
    plan->part_shift = bucket_bits - lp;
    return true;
}

PartSizes part_sizes(uint32_t dim, size_t n) {
    PartSizes z{};
    const size_t n_tiles = (n + PT_TILE - 1) / PT_TILE;
    const size_t np = n_tiles * PT_TILE;
    z.stage = np * 16;
    z.starts = n_tiles * (PT_MAX_PARTS + 1) * 4;
    z.pstart = (part_units(PT_MAX_PARTS, true) + 1) * 4;
    z.psum = n_tiles * PT_MAX_MULTI * (size_t)dim * 4;
    z.new_slot = np * 4;
    z.new_count = part_units(PT_MAX_PARTS, true) * 4;
    z.ngrad = np * (size_t)dim * 4;
    z.psize = PT_MAX_PARTS * 4;
    z.order = (part_units(PT_MAX_PARTS, true) + 2) * 4;  // slots, then {partitions, bucket mask} of its plan
    z.resv = PT_MAX_PARTS * 4;
    return z;
}

hipError_t part_init() {
    hipError_t e;
    if ((e = hipFuncSetAttribute(reinterpret_cast<const void*>(&part_tile_kernel<float>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, PT_LDS_FIXED + PT_MAX_PARTS * 4)) != hipSuccess) return e;
    if ((e = hipFuncSetAttribute(reinterpret_cast<const void*>(&part_tile_kernel<float4>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, PT_LDS_FIXED + PT_MAX_PARTS * 4)) != hipSuccess) return e;
    if ((e = hipFuncSetAttribute(reinterpret_cast<const void*>(&part_apply_kernel<float>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, PA_LDS)) != hipSuccess) return e;
    if ((e = hipFuncSetAttribute(reinterpret_cast<const void*>(&part_apply_kernel<float4>),
                                 hipFuncAttributeMaxDynamicSharedMemorySize, PA_LDS)) != hipSuccess) return e;
    return hipSuccess;
}

hipError_t launch_part_tile(const TableDev& t, const PartPlan& pl, const PartBufs& b, const uint64_t* keys,
                            const float* grads, const uint32_t* handles, hipStream_t s) {
    if ((t.dim % 4 == 0) && aligned16(grads))
        part_tile_kernel<float4><<<pl.n_tiles, PT_BLOCK, PT_LDS_FIXED + pl.P * 4, s>>>(
            t, keys, reinterpret_cast<const float4*>(grads), handles, pl.n, pl.P, pl.part_shift, b.stage, b.starts,
            reinterpret_cast<float4*>(b.psum), t.dim / 4);
    else
        part_tile_kernel<float><<<pl.n_tiles, PT_BLOCK, PT_LDS_FIXED + pl.P * 4, s>>>(
            t, keys, grads, handles, pl.n, pl.P, pl.part_shift, b.stage, b.starts, b.psum, t.dim);
    return hipGetLastError();
}

hipError_t launch_part_apply(const TableDev& t, const PartPlan& pl, const PartBufs& b, const float* grads, bool insert,
                             bool handles, bool verify, bool use_order, hipStream_t s) {
    const bool v4 = (t.dim % 4 == 0) && aligned16(grads);
    u32 pow2 = 1;
    while (pow2 < pl.n_tiles) pow2 <<= 1;
    ApplyArgs a{b.stage, b.starts, b.pstart, pl.n_tiles, pl.P, pl.n, pow2 / 2, b.new_slot, b.new_count,
                v4 ? t.dim / 4 : t.dim, insert ? 1 : 0, g_part_cap, handles ? 1 : 0, (handles && verify) ? 1 : 0,
                use_order ? b.order : nullptr, b.psize, b.resv};
    const u32 grid = part_units(pl.P, use_order);
    if (v4)
        part_apply_kernel<float4><<<grid, PA_BLOCK, PA_LDS, s>>>(t, reinterpret_cast<const float4*>(grads),
                                                                 reinterpret_cast<const float4*>(b.psum),
                                                                 reinterpret_cast<float4*>(b.ngrad), a);
    else
        part_apply_kernel<float><<<grid, PA_BLOCK, PA_LDS, s>>>(t, grads, b.psum, b.ngrad, a);
    return hipGetLastError();
}

hipError_t launch_part_insert(const TableDev& t, const PartPlan& pl, const PartBufs& b, const float* grads,
                              bool used_order, bool make_order, hipStream_t s) {
    const u32 units = part_units(pl.P, used_order);  // workgroups the apply kernel had
    const u32 grid = units + (make_order ? 8u : 0u);
    if ((t.dim % 4 == 0) && aligned16(grads))
        part_insert_kernel<float4><<<grid, PI_BLOCK, 0, s>>>(t, b.new_slot, reinterpret_cast<const float4*>(b.ngrad),
                                                             b.new_count, b.pstart, units, t.dim / 4, b.psize, b.order,
                                                             b.resv, pl.P, make_order ? 8u : 0u);
    else
        part_insert_kernel<float><<<grid, PI_BLOCK, 0, s>>>(t, b.new_slot, b.ngrad, b.new_count, b.pstart, units,
                                                            t.dim, b.psize, b.order, b.resv, pl.P, make_order ? 8u : 0u);
    return hipGetLastError();
}

}  // namespace pshbm

