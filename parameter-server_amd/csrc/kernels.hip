// HIP kernels of the HBM sparse table, written for gfx950 (64-wide wavefronts).
//
// Work decomposition used throughout: a wavefront handles a group of keys per round. Probing
// gives four lanes to a key — they read the four 16-byte slots of one 64-byte bucket with one
// dwordx4 load each and agree on the outcome with a ballot. Row traffic gives `row units` lanes
// to a key, so that consecutive lanes touch consecutive 16 bytes of a row or of the packed
// response.
#include "table.h"
#include "probe.h"
#include "rowops.h"

namespace pshbm {

namespace {

constexpr u32 WON_BIT = 0x80000000u;  // in a located slot index: this key claimed the slot in this launch
constexpr u32 ASSIGN_KEYS = 1024;     // keys per workgroup of assign_rows_kernel

// ---- row gather into the packed response -----------------------------------------------------
// `row` holds, in the lanes of group k, the row of key base + k (ROW_NONE = miss -> the weights a
// new key would start with: zeros, or init_weight() when the table draws them).
template <typename T>
__device__ __forceinline__ void gather_round(const TableDev& t, u32 row, u64 base, u32 cnt,
                                             T* __restrict__ out, u32 units, u32 stride_units,
                                             u64 m32, u32 lane, const u64* __restrict__ keys) {
    const T* rows = reinterpret_cast<const T*>(t.rows);
    const u32 total = cnt * units;
    for (u32 j0 = 0; j0 < total; j0 += 64) {
        u32 j = j0 + lane;
        bool on = j < total;
        u32 k = on ? div_small(j, m32) : 0u;
        u32 c = j - k * units;
        u32 r = __shfl(row, (int)(k * 4));
        if (on) {
            T v = vzero(T());
            if (r != ROW_NONE) {
                v = rows[(u64)r * stride_units + c];
            } else if (t.opt.init_range != 0.0f) {
                const u64 key = keys[base + k];
                if (key < KEY_DELETED) v = init_pulled(t, key, c, T());
            }
            out[base * units + j] = v;
        }
    }
}

template <typename T>
__global__ __launch_bounds__(BLOCK) void pull_kernel(TableDev t, const u64* __restrict__ keys,
                                                      u32 n, T* __restrict__ out,
                                                      uint8_t* __restrict__ hit,
                                                      u32* __restrict__ handles, u32 units,
                                                      u32 stride_units, u64 m32) {
    const u32 lane = threadIdx.x & 63u;
    const u32 grp = lane >> 2, sub = lane & 3u;
    const u64 wave = ((u64)blockIdx.x * BLOCK + threadIdx.x) >> 6;
    const u64 nwaves = ((u64)gridDim.x * BLOCK) >> 6;
    for (u64 base = wave * KEYS_PER_ROUND; base < n; base += nwaves * KEYS_PER_ROUND) {
        u64 i = base + grp;
        bool inb = i < n;
        u64 key = inb ? keys[i] : KEY_EMPTY;
        bool active = inb && key < KEY_DELETED;
        Found f = probe_find(t, key, active, grp, sub);
        if (hit && inb && sub == 0) hit[i] = f.row != ROW_NONE;
        if (handles && inb && sub == 0) handles[i] = f.row;  // the row, or ROW_NONE
        u32 cnt = (u32)((n - base) < KEYS_PER_ROUND ? (n - base) : KEYS_PER_ROUND);
        gather_round<T>(t, f.row, base, cnt, out, units, stride_units, m32, lane, keys);
    }
}

template <typename T>
__global__ __launch_bounds__(BLOCK) void gather_slots_kernel(TableDev t,
                                                              const u64* __restrict__ keys,
                                                              const u32* __restrict__ slot_idx,
                                                              u32 n, T* __restrict__ out,
                                                              uint8_t* __restrict__ hit,
                                                              u32* __restrict__ handles, u32 units,
                                                              u32 stride_units, u64 m32) {
    const u32 lane = threadIdx.x & 63u;
    const u32 grp = lane >> 2, sub = lane & 3u;
    const u64 wave = ((u64)blockIdx.x * BLOCK + threadIdx.x) >> 6;
    const u64 nwaves = ((u64)gridDim.x * BLOCK) >> 6;
    const u32 entry_rows = t.counters[CNT_ENTRY];
    for (u64 base = wave * KEYS_PER_ROUND; base < n; base += nwaves * KEYS_PER_ROUND) {
        u64 i = base + grp;
        u32 row = ROW_NONE;
        if (i < n) {
            u32 s = slot_idx[i];
            if (s != SLOT_NONE) row = reinterpret_cast<const u32*>(&t.slots[s])[2];
            if (row >= t.max_rows) row = ROW_NONE;
            if (hit && sub == 0) hit[i] = row < entry_rows;
            if (handles && sub == 0) handles[i] = row;
        }
        u32 cnt = (u32)((n - base) < KEYS_PER_ROUND ? (n - base) : KEYS_PER_ROUND);
        gather_round<T>(t, row, base, cnt, out, units, stride_units, m32, lane, keys);
    }
}

// ---- locate / claim ------------------------------------------------------------------------
template <bool kInsert>
__global__ __launch_bounds__(BLOCK) void locate_kernel(TableDev t, const u64* __restrict__ keys,
                                                        u32 n, u32* __restrict__ slot_out,
                                                        u32* __restrict__ idx_out,
                                                        u32* __restrict__ row_out,
                                                        u32* __restrict__ won_count,
                                                        int count_dups) {
    const u32 lane = threadIdx.x & 63u;
    const u32 grp = lane >> 2, sub = lane & 3u;
    const u64 wave = ((u64)blockIdx.x * BLOCK + threadIdx.x) >> 6;
    const u64 nwaves = ((u64)gridDim.x * BLOCK) >> 6;
    // the row count as it is when this operation begins (nothing in this launch changes it)
    if (kInsert && blockIdx.x == 0 && threadIdx.x == 0) t.counters[CNT_ENTRY] = t.counters[CNT_ROWS];
    for (u64 base = wave * KEYS_PER_ROUND; base < n; base += nwaves * KEYS_PER_ROUND) {
        u64 i = base + grp;
        bool inb = i < n;
        u64 key = inb ? keys[i] : KEY_EMPTY;
        bool active = inb && key < KEY_DELETED;
        {  // one addition per wavefront: a batch full of them must not queue up on one address
            const u64 bm = __ballot(inb && !active && sub == 0);
            if (bm && lane == (u32)__ffsll((unsigned long long)bm) - 1u)
                atomicAdd(&t.counters[CNT_BADKEY], (u32)__popcll(bm));
        }
        u32 slot = SLOT_NONE;
        u32 row = ROW_NONE;
        bool dup = false;
        if constexpr (!kInsert) {
            Found f = probe_find(t, key, active, grp, sub);
            slot = f.slot;
            row = f.row;
            dup = f.slot != SLOT_NONE;
        } else {
            const Located l = find_or_claim(t, key, active, grp, sub, row_out != nullptr);
            slot = l.slot;
            row = l.row;
            dup = l.dup;
            // The group that claimed the slot only marks it and counts itself in its 1024-key
            // block: rows are handed out afterwards by assign_rows_kernel. (One shared row counter
            // bumped from here costs a device-scope atomic on one address per wavefront, which
            // serialises: 1.5 ms for 200,000 inserts.)
            // (Nor does every winner count itself: additions to one address are resolved one
            // after the other, about 120 ns each, and the 1024 keys of a block are probed at about
            // the same time. The 16 keys of a round lie in one block: one addition per wavefront.)
            static_assert(ASSIGN_KEYS % KEYS_PER_ROUND == 0, "a round's keys share a block");
            const u64 wm = __ballot(l.won && sub == 0);
            if (wm) {
                if (lane == (u32)__ffsll((unsigned long long)wm) - 1u)
                    atomicAdd(&won_count[base / ASSIGN_KEYS], (u32)__popcll(wm));
                if (l.won && sub == 0) slot |= WON_BIT;
            }
        }
        if (inb && sub == 0) {
            slot_out[i] = slot;
            if (idx_out) idx_out[i] = (u32)i;
            if (row_out) row_out[i] = row;
        }
        if (count_dups) {
            const u64 dm = __ballot(inb && sub == 0 && dup);
            if (dm && lane == (u32)__ffsll((unsigned long long)dm) - 1u)
                atomicAdd(&t.counters[CNT_DUP], (u32)__popcll(dm));
        }
    }
}

// Dense row ids for the slots that locate_kernel<true> claimed (slot_idx[i] carries WON_BIT).
// Workgroup b owns keys [b * ASSIGN_KEYS, (b+1) * ASSIGN_KEYS); won_count[b] is how many of them
// won. Its first row is CNT_ENTRY + the counts of the workgroups before it (summed here: a few
// thousand words at most), then winners are numbered in (round, thread) order with ballots. The
// rows are initialised, row_keys and the slot's row word are written, WON_BIT is cleared.
// Workgroup 0 publishes the new row count; every workgroup zeroes its word of `won_next`, the
// array the next operation counts into. Rows past the capacity raise CNT_OVERFLOW and stay unset.
__global__ __launch_bounds__(BLOCK) void assign_rows_kernel(TableDev t, const u64* __restrict__ keys,
                                                             u32 n, u32* __restrict__ slot_idx,
                                                             u32* __restrict__ row_out,
                                                             const u32* __restrict__ won_count,
                                                             u32* __restrict__ won_next, u32 won_words,
                                                             u32 n_blocks, int init_rows) {
    __shared__ u32 red[BLOCK / 64];
    __shared__ u32 wave_cnt[ASSIGN_KEYS / BLOCK][BLOCK / 64];
    const u32 b = blockIdx.x, tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    for (u32 x = b * BLOCK + tid; x < won_words; x += gridDim.x * BLOCK) won_next[x] = 0;
    const u32 mine = won_count[b];
    if (mine == 0 && b != 0) return;  // block-uniform
    // winners in the workgroups before this one (workgroup 0: in all of them, for the new total)
    const u32 upto = b == 0 ? n_blocks : b;
    u32 part = 0;
    for (u32 x = tid; x < upto; x += BLOCK) part += won_count[x];
    for (u32 off = 32; off >= 1; off >>= 1) part += __shfl_down(part, off);
    if (lane == 0) red[w] = part;
    __syncthreads();
    u32 sum = 0;
    for (u32 x = 0; x < BLOCK / 64; ++x) sum += red[x];
    const u32 entry = t.counters[CNT_ENTRY];
    if (b == 0) {
        if (tid == 0) {
            t.counters[CNT_ROWS] = entry + sum;
            if (entry + sum > t.max_rows) t.counters[CNT_OVERFLOW] = 1u;
            publish_rows(t, entry + sum);
        }
        if (mine == 0) return;
        sum = 0;
    }
    const u32 first_row = entry + sum;
    // number the winners of this workgroup
    u32 s[ASSIGN_KEYS / BLOCK];
    u32 before[ASSIGN_KEYS / BLOCK];
    const u64 lt_mask = (1ull << lane) - 1ull;
#pragma unroll
    for (u32 j = 0; j < ASSIGN_KEYS / BLOCK; ++j) {
        const u64 i = (u64)b * ASSIGN_KEYS + j * BLOCK + tid;
        s[j] = i < n ? slot_idx[i] : SLOT_NONE;
        const bool won = s[j] != SLOT_NONE && (s[j] & WON_BIT);
        const u64 m = __ballot(won);
        before[j] = (u32)__popcll(m & lt_mask);
        if (lane == 0) wave_cnt[j][w] = (u32)__popcll(m);
    }
    __syncthreads();
    u32 run = 0;
#pragma unroll
    for (u32 j = 0; j < ASSIGN_KEYS / BLOCK; ++j) {
        u32 my_base = run;
        for (u32 x = 0; x < BLOCK / 64; ++x) {
            if (x < w) my_base += wave_cnt[j][x];
            run += wave_cnt[j][x];
        }
        const bool won = s[j] != SLOT_NONE && (s[j] & WON_BIT);
        if (!won) continue;
        const u64 i = (u64)b * ASSIGN_KEYS + j * BLOCK + tid;
        const u32 slot = s[j] & ~WON_BIT;
        slot_idx[i] = slot;
        const u32 rid = first_row + my_base + before[j];
        if (rid >= t.max_rows) {  // does not fit: the caller rolls the batch back
            if (row_out) row_out[i] = ROW_NONE;
            continue;
        }
        if (row_out) row_out[i] = rid;
        reinterpret_cast<u32*>(&t.slots[slot])[2] = rid;
        t.row_keys[rid] = keys[i];
        if (init_rows) {
            float4* r4 = reinterpret_cast<float4*>(t.rows + (u64)rid * t.stride_f);
            for (u32 c = 0; c < t.stride_f / 4; ++c) {
                const u32 f = c * 4;
                r4[c] = make_float4(init_float(t, keys[i], f), init_float(t, keys[i], f + 1),
                                    init_float(t, keys[i], f + 2), init_float(t, keys[i], f + 3));
            }
        }
    }
}

__global__ __launch_bounds__(BLOCK) void rollback_kernel(TableDev t, const u32* __restrict__ slot_idx,
                                                          u32 n, u32 first_new_row) {
    u64 i = (u64)blockIdx.x * BLOCK + threadIdx.x;
    if (i == 0) {
        t.counters[CNT_ROWS] = first_new_row;
        t.counters[CNT_OVERFLOW] = 0u;
    }
    if (i >= n) return;
    u32 s = slot_idx[i];
    if (s == SLOT_NONE) return;
    u32 r = reinterpret_cast<const u32*>(&t.slots[s])[2];
    if (r == ROW_NONE || r >= first_new_row)
        t.slots[s] = make_uint4(0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu, 0xFFFFFFFFu);
}

__global__ __launch_bounds__(BLOCK) void fill_u32_kernel(u32* p, u64 n, u32 v) {
    for (u64 i = (u64)blockIdx.x * BLOCK + threadIdx.x; i < n; i += (u64)gridDim.x * BLOCK) p[i] = v;
}

// ---- duplicate aggregation + update over row-sorted pairs --------------------------------------
// Each wavefront owns `wch` consecutive sorted positions (a chunk). It copies the chunk's row ids
// and the gradient rows they point to into LDS (16 independent row loads per lane in flight),
// lists the starts of the runs of equal row ids with ballots, and then gives each run to one group
// of `lp` lanes, which adds the run's rows in sorted order, one LDS read per row. A run longer
// than 2 P rows is added by all P groups together (strided, then a shuffle tree). A run that
// begins and ends inside the chunk is complete: its sum is applied to the table row, four runs
// per lane group at a time so that the row loads of different runs overlap. A run that crosses a
// chunk border leaves a partial sum in part_val (entry 0: the run that entered from the left,
// entry 1: the run that leaves to the right) for fixup_kernel to join.
// part_hdr[w] = {row of entry 0, flags of entry 0 (1 present, 2 run ends in this chunk),
//               row of entry 1, flags of entry 1 (1 present)}.
// LDS per wavefront: wch * lp_full elements of T, then three arrays of wch + 1 words (row ids;
// batch indices, later one action word per run; run starts).
constexpr int SEG_BLOCK = 128;  // 2 wavefronts

__device__ __forceinline__ void wave_sync() {
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

__device__ __forceinline__ float vshfl_down(float v, u32 d) { return __shfl_down(v, d); }
__device__ __forceinline__ float4 vshfl_down(float4 v, u32 d) {
    return make_float4(__shfl_down(v.x, d), __shfl_down(v.y, d), __shfl_down(v.z, d),
                       __shfl_down(v.w, d));
}

// Applies the sums that segreduce_kernel left in LDS (first row of each run whose action word is
// set) to the table rows, FB runs per lane group at a time. STATES = optimizer state blocks.
template <typename T, int KIND, u32 FB>
__device__ __forceinline__ void apply_runs(const TableDev& t, const T* s_val, const u32* s_row,
                                           const u32* s_act, const u32* s_start, u32 nruns, u32 P,
                                           u32 g, u32 c, bool lane_on, u32 lp_full, u32 units,
                                           u32 col) {
    constexpr int N = sizeof(T) / 4;
    constexpr int STATES = states_of<KIND>();
    T* rows = reinterpret_cast<T*>(t.rows);
    const u32 stride_units = t.stride_f / N;
    for (u32 j0 = 0; j0 < nruns; j0 += FB * P) {
        u32 row[FB], st[FB];
        T wv[FB], av[STATES >= 1 ? FB : 1], bv[STATES >= 2 ? FB : 1];
#pragma unroll
        for (u32 k = 0; k < FB; ++k) {
            const u32 j = j0 + k * P + g;
            row[k] = ROW_NONE;
            st[k] = 0;
            if (lane_on && j < nruns && s_act[j]) {
                st[k] = s_start[j];
                const u32 r = s_row[st[k]];
                if (r < t.max_rows) row[k] = r;
            }
        }
#pragma unroll
        for (u32 k = 0; k < FB; ++k) {
            if (row[k] == ROW_NONE) continue;
            const T* r = rows + (u64)row[k] * stride_units + col;
            wv[k] = r[0];
            if constexpr (STATES >= 1) av[k] = r[units];
            if constexpr (STATES >= 2) bv[k] = r[2 * units];
        }
#pragma unroll
        for (u32 k = 0; k < FB; ++k) {
            if (row[k] == ROW_NONE) continue;
            T gs = s_val[st[k] * lp_full + c];
            T a0 = vzero(T()), b0 = vzero(T());
            if constexpr (STATES >= 1) a0 = av[k];
            if constexpr (STATES >= 2) b0 = bv[k];
            float* gp = reinterpret_cast<float*>(&gs);
            float* wp = reinterpret_cast<float*>(&wv[k]);
            float* ap = reinterpret_cast<float*>(&a0);
            float* bp = reinterpret_cast<float*>(&b0);
#pragma unroll
            for (int e = 0; e < N; ++e) opt_step<KIND>(t.opt, gp[e], wp[e], ap[e], bp[e]);
            T* r = rows + (u64)row[k] * stride_units + col;
            if (t.dirty && col == 0) t.dirty[row[k]] = 1;
            r[0] = wv[k];
            if constexpr (STATES >= 1) r[units] = a0;
            if constexpr (STATES >= 2) r[2 * units] = b0;
        }
    }
}

template <typename T>
__global__ __launch_bounds__(SEG_BLOCK) void segreduce_kernel(
    TableDev t, const u32* __restrict__ srow, const u32* __restrict__ sidx, u32 n,
    const T* __restrict__ grads, uint4* __restrict__ part_hdr, T* __restrict__ part_val, u32 units,
    u32 lp_full, u32 P, u32 wch, u32 n_chunks, u32 val_bytes, u32 arr_bytes) {
    extern __shared__ uint4 seg_lds[];
    const u32 lane = threadIdx.x & 63u;
    const u32 wv = threadIdx.x >> 6;
    const u32 w = blockIdx.x * (SEG_BLOCK / 64) + wv;
    if (w >= n_chunks) return;  // no workgroup barriers below
    // a sort that gave up (a tile's bounded wait ran out) left pairs that are not grouped by row:
    // nothing is applied, the host reports the push as failed
    if (t.counters[CNT_SORT_ERR]) return;
    char* base = reinterpret_cast<char*>(seg_lds) + (size_t)wv * (val_bytes + 3 * arr_bytes);
    T* s_val = reinterpret_cast<T*>(base);
    u32* s_row = reinterpret_cast<u32*>(base + val_bytes);
    u32* s_aux = reinterpret_cast<u32*>(base + val_bytes + arr_bytes);
    u32* s_start = reinterpret_cast<u32*>(base + val_bytes + 2 * arr_bytes);

    const u32 col0 = blockIdx.y * 64u;
    const u32 lp = (units - col0) < 64u ? (units - col0) : 64u;
    const u32 g = lane / lp_full;
    const u32 c = lane - g * lp_full;
    const bool lane_on = g < P && c < lp;
    const u32 cs = w * wch;
    const u32 cnt = (n - cs) < wch ? (n - cs) : wch;

    // row ids and batch indices of the chunk
    for (u32 pl = lane; pl < wch; pl += 64) {
        u32 sl = SLOT_NONE, ix = 0;
        if (pl < cnt) {
            sl = srow[cs + pl];
            ix = sidx[cs + pl];
        }
        s_row[pl] = sl;
        s_aux[pl] = ix;
    }
    const u32 first_row = srow[cs];
    const u32 last_row = srow[cs + cnt - 1];
    const bool open_left = cs > 0 && srow[cs - 1] == first_row;
    const u32 after = cs + cnt < n ? srow[cs + cnt] : SLOT_NONE;
    wave_sync();

    // gradient rows into LDS: position r * P + g in round r
    {
        T v[SEG_ROUNDS];
#pragma unroll
        for (u32 r = 0; r < SEG_ROUNDS; ++r) {
            const u32 pl = r * P + g;
            v[r] = vzero(T());
            if (lane_on && pl < cnt && s_row[pl] != SLOT_NONE)
                v[r] = grads[(u64)s_aux[pl] * units + col0 + c];
        }
#pragma unroll
        for (u32 r = 0; r < SEG_ROUNDS; ++r) {
            const u32 pl = r * P + g;
            if (lane_on) s_val[pl * lp_full + c] = v[r];
        }
    }
    wave_sync();

    // run starts; unfound keys (SLOT_NONE) sort last and form no run
    u32 nruns = 0, nreal = 0;
    for (u32 k0 = 0; k0 < wch; k0 += 64) {
        const u32 pl = k0 + lane;
        u32 sl = SLOT_NONE, pv = SLOT_NONE;
        if (pl < wch) {
            sl = s_row[pl];
            if (pl > 0) pv = s_row[pl - 1];
        }
        const bool real = sl != SLOT_NONE;
        const bool head = real && (pl == 0 || pv != sl);
        const u64 hm = __ballot(head);
        if (head) s_start[nruns + (u32)__popcll(hm & ((1ull << lane) - 1ull))] = pl;
        nruns += (u32)__popcll(hm);
        nreal += (u32)__popcll(__ballot(real));
    }
    if (lane == 0) s_start[nruns] = nreal;
    wave_sync();

    // sums of the runs. A sum that can be applied goes back to LDS in the run's first row and the
    // run's action word becomes 1; a sum that crosses a border goes to part_val.
    bool my_l = false, my_le = false, my_r = false;
    auto classify = [&](u32 j, u32 st, u32 en, T acc) {
        const u32 sl = s_row[st];
        const bool first_run = open_left && j == 0;
        const bool last_open = en == cnt && after == sl;
        u32 act = 0;
        if (first_run) {
            part_val[((u64)w * 2 + 0) * units + col0 + c] = acc;
            my_l = true;
            my_le = !last_open;
        } else if (last_open) {
            part_val[((u64)w * 2 + 1) * units + col0 + c] = acc;
            my_r = true;
        } else {
            s_val[st * lp_full + c] = acc;
            act = 1;
        }
        if (c == 0) s_aux[j] = act;
    };
    u32 top = 1;
    while (top < P) top <<= 1;
    const u32 long_run = 2 * P;
    for (u32 j0 = 0; j0 < nruns; j0 += P) {
        const u32 j = j0 + g;
        const bool have = lane_on && j < nruns;
        u32 st = 0, en = 0;
        if (have) {
            st = s_start[j];
            en = s_start[j + 1];
        }
        const bool is_long = P > 1 && en - st > long_run;
        if (have && !is_long) {
            T acc = vzero(T());
            for (u32 q = st; q < en; ++q) acc = vadd(acc, s_val[q * lp_full + c]);
            classify(j, st, en, acc);
        }
        u64 lm = __ballot(have && is_long && c == 0);
        while (lm) {
            const u32 src = (u32)__ffsll((unsigned long long)lm) - 1u;
            lm &= lm - 1;
            const u32 jj = __shfl(j, (int)src), s2 = __shfl(st, (int)src), e2 = __shfl(en, (int)src);
            T a = vzero(T());
            if (lane_on)
                for (u32 q = s2 + g; q < e2; q += P) a = vadd(a, s_val[q * lp_full + c]);
            for (u32 off = top >> 1; off >= 1; off >>= 1) {
                T o = vshfl_down(a, off * lp_full);
                if (g + off < P) a = vadd(a, o);
            }
            if (lane_on && g == 0) classify(jj, s2, e2, a);
        }
    }
    wave_sync();

    // optimizer step on the rows of the complete runs; a lane group holds as many runs at once
    // as registers allow, so that their row loads overlap
    const u32 col = col0 + c;
    switch (t.opt.kind) {
        case 0:
            apply_runs<T, 0, SEG_ROUNDS>(t, s_val, s_row, s_aux, s_start, nruns, P, g, c, lane_on,
                                         lp_full, units, col);
            break;
        case 1:
            apply_runs<T, 1, SEG_ROUNDS>(t, s_val, s_row, s_aux, s_start, nruns, P, g, c, lane_on,
                                         lp_full, units, col);
            break;
        case 2:
            apply_runs<T, 2, SEG_ROUNDS / 2>(t, s_val, s_row, s_aux, s_start, nruns, P, g, c, lane_on,
                                             lp_full, units, col);
            break;
        case 3:
            apply_runs<T, 3, SEG_ROUNDS / 4>(t, s_val, s_row, s_aux, s_start, nruns, P, g, c, lane_on,
                                             lp_full, units, col);
            break;
        default:
            apply_runs<T, 4, SEG_ROUNDS / 4>(t, s_val, s_row, s_aux, s_start, nruns, P, g, c, lane_on,
                                             lp_full, units, col);
            break;
    }

    const bool l_present = __any(my_l) != 0, l_ends = __any(my_le) != 0, r_present = __any(my_r) != 0;
    if (lane == 0 && blockIdx.y == 0)
        part_hdr[w] = make_uint4(first_row, (l_present ? 1u : 0u) | (l_ends ? 2u : 0u), last_row,
                                 r_present ? 1u : 0u);
}

// Sum of p[x * stride] for x = first, first + step, ... < end, four loads in flight at a time (the
// order of the additions is fixed by first / end / step alone).
template <typename T>
__device__ __forceinline__ T strided_sum(const T* __restrict__ p, u64 first, u64 end, u32 step, u64 stride) {
    T a0 = vzero(T()), a1 = vzero(T()), a2 = vzero(T()), a3 = vzero(T());
    u64 x = first;
    for (; x + 3 * (u64)step < end; x += 4 * (u64)step) {
        const T v0 = p[x * stride], v1 = p[(x + step) * stride], v2 = p[(x + 2 * (u64)step) * stride],
                v3 = p[(x + 3 * (u64)step) * stride];
        a0 = vadd(a0, v0);
        a1 = vadd(a1, v1);
        a2 = vadd(a2, v2);
        a3 = vadd(a3, v3);
    }
    for (; x < end; x += step) a0 = vadd(a0, p[x * stride]);
    return vadd(vadd(a0, a1), vadd(a2, a3));
}

// A key repeated hundreds of thousands of times in a batch spans thousands of chunks. So that the
// wavefront that joins its partial sums need not visit every one of them, a first pass looks at
// windows of 64 chunks: if all 64 chunks of a window lie inside one run (each chunk is a single run
// that is open on both sides), their partial sums are added up into win_val[window] and
// win_row[window] names the run's row; any other window gets SLOT_NONE.
constexpr u32 WINDOW = 64;

template <typename T>
__global__ __launch_bounds__(BLOCK) void fixup_windows_kernel(const uint4* __restrict__ part_hdr,
                                                               const T* __restrict__ part_val,
                                                               u32* __restrict__ win_row,
                                                               T* __restrict__ win_val, u32 units,
                                                               u32 lp_full, u32 P, u32 n_chunks,
                                                               u32 n_windows) {
    const u32 lane = threadIdx.x & 63u;
    const u32 v = blockIdx.x * (BLOCK / 64) + (threadIdx.x >> 6);
    if (v >= n_windows) return;
    const u32 x = v * WINDOW + lane;
    bool through = false;
    u32 sl = SLOT_NONE;
    if (x < n_chunks) {
        const uint4 h = part_hdr[x];
        through = (h.y & 1u) && !(h.y & 2u) && !(h.w & 1u);
        sl = h.x;
    }
    const u32 s0 = __shfl(sl, 0);
    const bool whole = __ballot(through && sl == s0) == ~0ull;
    if (!whole) {
        if (lane == 0 && blockIdx.y == 0) win_row[v] = SLOT_NONE;
        return;
    }
    const u32 col0 = blockIdx.y * 64u;
    const u32 lp = (units - col0) < 64u ? (units - col0) : 64u;
    const u32 g = lane / lp_full;
    const u32 c = lane - g * lp_full;
    const bool lane_on = g < P && c < lp;
    const u32 col = col0 + c;
    T acc = vzero(T());
    if (lane_on) acc = strided_sum(part_val + col, (u64)v * WINDOW + g, (u64)(v + 1) * WINDOW, P, 2 * (u64)units);
    u32 top = 1;
    while (top < P) top <<= 1;
    for (u32 off = top >> 1; off >= 1; off >>= 1) {
        T o = vshfl_down(acc, off * lp_full);
        if (g + off < P) acc = vadd(acc, o);
    }
    if (lane_on && g == 0) win_val[(u64)v * units + col] = acc;
    if (lane == 0 && blockIdx.y == 0) win_row[v] = s0;
}

// Joins the partial sums of runs that cross chunk borders. One wavefront per chunk: if a run
// leaves that chunk to the right, the wavefront finds where the run ends (the first following
// chunk whose left entry is marked as the run's end; whole windows of the run are skipped through
// win_row), its P lane groups add, in a strided fashion, the left entries of the chunks in
// between -- window sums where a window lies wholly inside the run --, a shuffle tree joins the P
// sums, and group 0 applies the step. The order of the additions depends only on the chunk
// layout, so results repeat from run to run.
template <typename T>
__global__ __launch_bounds__(BLOCK) void fixup_kernel(TableDev t, const uint4* __restrict__ part_hdr,
                                                       const T* __restrict__ part_val,
                                                       const u32* __restrict__ win_row,
                                                       const T* __restrict__ win_val, u32 units,
                                                       u32 lp_full, u32 P, u32 n_chunks, u32 n_windows) {
    const u32 lane = threadIdx.x & 63u;
    const u32 w = blockIdx.x * (BLOCK / 64) + (threadIdx.x >> 6);
    if (w >= n_chunks) return;
    if (t.counters[CNT_SORT_ERR]) return;  // the sort gave up: segreduce_kernel wrote no partial sums
    const uint4 h = part_hdr[w];
    if (!(h.w & 1u)) return;  // wave-uniform
    const u32 col0 = blockIdx.y * 64u;
    const u32 lp = (units - col0) < 64u ? (units - col0) : 64u;
    const u32 g = lane / lp_full;
    const u32 c = lane - g * lp_full;
    const bool lane_on = g < P && c < lp;
    const u32 col = col0 + c;
    // last chunk of the run
    u32 last = w;
    u32 x0 = w + 1;
    bool found = false;
    while (!found && x0 < n_chunks) {
        // the rest of x0's window, a header per lane
        const u32 wend = (x0 / WINDOW + 1) * WINDOW < n_chunks ? (x0 / WINDOW + 1) * WINDOW : n_chunks;
        const u32 x = x0 + lane;
        bool ends = false, brk = false;
        if (x < wend) {
            const uint4 hx = part_hdr[x];
            const bool same = (hx.y & 1u) && hx.x == h.z;
            ends = same && (hx.y & 2u);
            brk = !same;
        }
        const u64 em = __ballot(ends), bm = __ballot(brk);
        const u64 any = em | bm;
        if (any) {
            const u32 f = (u32)__ffsll((unsigned long long)any) - 1u;
            last = ((em >> f) & 1ull) ? x0 + f : x0 + f - 1u;
            found = true;
            break;
        }
        last = wend - 1u;
        x0 = wend;
        // whole windows of this run, 64 window words per step
        while (x0 < n_chunks) {
            const u32 vv = x0 / WINDOW + lane;
            const bool mine = vv < n_windows && win_row[vv] == h.z;
            const u64 nm = ~__ballot(mine);
            const u32 k = nm ? (u32)__ffsll((unsigned long long)nm) - 1u : 64u;
            if (k) {
                x0 += k * WINDOW;
                last = x0 - 1u;
            }
            if (k < 64u) break;
        }
    }
    // sum: R entry of w, then the L entries of w+1 .. last
    const u64 A = (u64)w + 1, B = last;
    const u64 fs = (A + WINDOW - 1) / WINDOW * WINDOW;  // first window start at or after A
    const u64 fe = B / WINDOW * WINDOW;                 // start of B's window
    T acc = vzero(T());
    if (lane_on) {
        if (g == 0) acc = part_val[((u64)w * 2 + 1) * units + col];
        if (n_windows == 0 || fs >= fe) {  // no window sums were made, or no whole window inside
            acc = vadd(acc, strided_sum(part_val + col, A + g, B + 1, P, 2 * (u64)units));
        } else {
            acc = vadd(acc, strided_sum(part_val + col, A + g, fs, P, 2 * (u64)units));
            acc = vadd(acc, strided_sum(win_val + col, fs / WINDOW + g, fe / WINDOW, P, (u64)units));
            acc = vadd(acc, strided_sum(part_val + col, fe + g, B + 1, P, 2 * (u64)units));
        }
    }
    u32 top = 1;
    while (top < P) top <<= 1;
    for (u32 off = top >> 1; off >= 1; off >>= 1) {
        T o = vshfl_down(acc, off * lp_full);
        if (g + off < P) acc = vadd(acc, o);
    }
    if (lane_on && g == 0) finalize<T>(t, h.z, col, units, acc);
}

// ---- a whole push in one launch, for small batches (the kernel takes up to 1024 keys) -----------
// Small batches are bound by launches, not by work, so one workgroup of 1024 threads does what the
// chain of kernels above does: (1) four lanes per key find the key or claim a slot for it;
// (2) thread i numbers key i's claim (a prefix sum over the workgroup), the new rows are
// initialised and the later occurrences of a new key read its row from its slot; (3) thread i
// ranks pair (row, i) among all pairs by comparing with every other one (n <= 1024: about a
// thousand LDS reads) and puts it at its place -- the pairs are then sorted by row, equal rows in
// batch order; (4) the starts of the runs of equal rows are listed; (5) groups of lanes, one lane
// per 4 or 16 bytes of a gradient row, add up a run each in batch order and take the optimizer
// step. A run of more than SMALL_LONG rows is added by all groups together: strided partial sums,
// then added in group order.
constexpr u32 SMALL_PUSH = 1024, SMALL_LONG = 32;

__device__ __forceinline__ u32 block_scan_1024(u32 v, u32 tid, u32* wave_sums, u32* total) {
    const u32 lane = tid & 63u, w = tid >> 6;
    u32 incl = v;
    for (u32 off = 1; off < 64; off <<= 1) {
        const u32 o = __shfl_up(incl, off);
        if (lane >= off) incl += o;
    }
    if (lane == 63) wave_sums[w] = incl;
    __syncthreads();
    u32 before = 0, all = 0;
    for (u32 x = 0; x < SMALL_PUSH / 64; ++x) {
        const u32 c = wave_sums[x];
        if (x < w) before += c;
        all += c;
    }
    *total = all;
    __syncthreads();  // wave_sums may be used again
    return before + incl - v;
}

template <typename T>
__global__ __launch_bounds__(SMALL_PUSH) void push_small_kernel(TableDev t, const u64* __restrict__ keys,
                                                                const T* __restrict__ grads, u32 n,
                                                                int insert, u32 units) {
    __shared__ u32 s_slot[SMALL_PUSH];                       // per key, batch order
    __shared__ __align__(16) u32 s_row[SMALL_PUSH];
    __shared__ u32 q_row[SMALL_PUSH], q_idx[SMALL_PUSH];    // pairs sorted by (row, batch index)
    __shared__ u32 heads[SMALL_PUSH + 1];                   // starts of the runs; heads[nruns] = their end
    __shared__ u32 longs[SMALL_PUSH / SMALL_LONG + 1];      // runs added by the whole workgroup
    __shared__ u32 new_idx[SMALL_PUSH];  // batch index of the k-th key inserted by this call
    __shared__ u32 wave_sums[SMALL_PUSH / 64];
    __shared__ u32 n_long;
    __shared__ T part[SMALL_PUSH];
    const u32 tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    const u32 grp = lane >> 2, sub = lane & 3u;
    const u32 entry = t.counters[CNT_ROWS];
    if (tid == 0) n_long = 0;

    // 1. find or claim: 256 keys per round
    for (u32 r0 = 0; r0 < n; r0 += SMALL_PUSH / 4) {
        const u32 i = r0 + w * KEYS_PER_ROUND + grp;
        const bool inb = i < n;
        const u64 key = inb ? keys[i] : KEY_EMPTY;
        const bool active = inb && key < KEY_DELETED;
        const u64 bm = __ballot(inb && !active && sub == 0);
        if (bm && lane == (u32)__ffsll((unsigned long long)bm) - 1u)
            atomicAdd(&t.counters[CNT_BADKEY], (u32)__popcll(bm));
        u32 slot = SLOT_NONE, row = ROW_NONE;
        if (insert) {
            const Located l = find_or_claim(t, key, active, grp, sub, true);
            slot = l.slot;
            row = l.row;
            if (l.won) slot |= WON_BIT;
        } else {
            const Found f = probe_find(t, key, active, grp, sub);
            slot = f.slot;
            row = f.row;
        }
        if (inb && sub == 0) {
            s_slot[i] = slot;
            s_row[i] = row;
        }
    }
    __syncthreads();

    // 2. rows for the claims, in batch order
    const bool won = tid < n && s_slot[tid] != SLOT_NONE && (s_slot[tid] & WON_BIT);
    u32 n_won = 0;
    const u32 rank = block_scan_1024(won ? 1u : 0u, tid, wave_sums, &n_won);
    if (won) {
        const u32 rid = entry + rank;
        const u32 slot = s_slot[tid] & ~WON_BIT;
        s_slot[tid] = slot;
        if (rid < t.max_rows) {
            reinterpret_cast<u32*>(&t.slots[slot])[2] = rid;
            t.row_keys[rid] = keys[tid];
            s_row[tid] = rid;
        } else {  // does not fit (the host rules this out before it chooses this kernel)
            s_row[tid] = ROW_NONE;
        }
        new_idx[rank] = tid;
    }
    if (tid == 0 && insert) {
        t.counters[CNT_ENTRY] = entry;
        t.counters[CNT_ROWS] = entry + n_won;
        if (entry + n_won > t.max_rows) t.counters[CNT_OVERFLOW] = 1u;
        publish_rows(t, entry + n_won);
    }
    __threadfence();
    __syncthreads();
    if (n_won) {
        // a later occurrence of a key claimed by this batch: the row is in the slot now
        if (tid < n && s_row[tid] == ROW_PENDING)
            s_row[tid] = __hip_atomic_load(reinterpret_cast<u32*>(&t.slots[s_slot[tid]]) + 2, __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_AGENT);
        // fresh rows: initial weights, initial optimizer state
        const u32 per = t.stride_f;
        for (u32 e = tid; e < n_won * per; e += SMALL_PUSH) {
            const u32 k = e / per, f = e - k * per;
            const u32 i = new_idx[k];
            const u32 rid = s_row[i];
            if (rid != ROW_NONE) t.rows[(u64)rid * per + f] = init_float(t, keys[i], f);
        }
        __threadfence();
        __syncthreads();
    }

    // 3. place of pair (row, i) among the pairs: those with a smaller row, or the same row earlier
    // (four rows per LDS read; the entries past n hold ROW_NONE and count for nobody)
    if (tid >= n) s_row[tid] = ROW_NONE;
    __syncthreads();
    if (tid < n) {
        const u32 mine = s_row[tid];
        const uint4* rows4 = reinterpret_cast<const uint4*>(s_row);
        u32 pos = 0;
#pragma unroll 4
        for (u32 j = 0; j < n; j += 4) {
            const uint4 o = rows4[j >> 2];
            pos += (o.x < mine || (o.x == mine && j < tid)) ? 1u : 0u;
            pos += (o.y < mine || (o.y == mine && j + 1 < tid)) ? 1u : 0u;
            pos += (o.z < mine || (o.z == mine && j + 2 < tid)) ? 1u : 0u;
            pos += (o.w < mine || (o.w == mine && j + 3 < tid)) ? 1u : 0u;
        }
        q_row[pos] = mine;
        q_idx[pos] = tid;
    }
    __syncthreads();

    // 4. run starts; keys that are not stored (ROW_NONE, the largest value) come last and form no run
    const bool real = tid < n && q_row[tid] < t.max_rows;
    const bool head = real && (tid == 0 || q_row[tid - 1] != q_row[tid]);
    u32 nruns = 0, nreal = 0;
    const u32 hpos = block_scan_1024(head ? 1u : 0u, tid, wave_sums, &nruns);
    (void)block_scan_1024(real ? 1u : 0u, tid, wave_sums, &nreal);
    if (head) heads[hpos] = tid;
    if (tid == 0) heads[nruns] = nreal;
    __syncthreads();
    if (tid < nruns && heads[tid + 1] - heads[tid] > SMALL_LONG) longs[atomicAdd(&n_long, 1u)] = tid;
    __syncthreads();

    // 5. sums and optimizer steps, 64 columns (of T) at a time
    for (u32 col0 = 0; col0 < units; col0 += 64) {
        const u32 lp = (units - col0) < 64u ? (units - col0) : 64u;  // lanes per row
        const u32 G = SMALL_PUSH / lp;                               // lane groups
        const u32 g = tid / lp, c = tid - g * lp;
        const u32 col = col0 + c;
        if (g < G) {
            for (u32 j = g; j < nruns; j += G) {
                const u32 st = heads[j], en = heads[j + 1];
                if (en - st > SMALL_LONG) continue;
                T a0 = vzero(T()), a1 = vzero(T());
                u32 q = st;
                for (; q + 1 < en; q += 2) {  // two loads in flight; the order of additions is fixed
                    const T v0 = grads[(u64)q_idx[q] * units + col];
                    const T v1 = grads[(u64)q_idx[q + 1] * units + col];
                    a0 = vadd(a0, v0);
                    a1 = vadd(a1, v1);
                }
                if (q < en) a0 = vadd(a0, grads[(u64)q_idx[q] * units + col]);
                finalize<T>(t, q_row[st], col, units, vadd(a0, a1));
            }
        }
        const u32 nl = n_long;
        for (u32 x = 0; x < nl; ++x) {  // workgroup-uniform
            const u32 j = longs[x];  // in no particular order: the runs are of different rows
            const u32 st = heads[j], en = heads[j + 1];
            T a = vzero(T());
            if (g < G)
                for (u32 q = st + g; q < en; q += G) a = vadd(a, grads[(u64)q_idx[q] * units + col]);
            __syncthreads();
            if (g < G) part[g * lp + c] = a;
            __syncthreads();
            if (g == 0) {
                T sum = vzero(T());
                const u32 used = (en - st) < G ? (en - st) : G;
                for (u32 y = 0; y < used; ++y) sum = vadd(sum, part[y * lp + c]);
                finalize<T>(t, q_row[st], col, units, sum);
            }
        }
        __syncthreads();
    }
}

template <typename T>
__global__ __launch_bounds__(BLOCK) void update_unique_kernel(TableDev t,
                                                               const u32* __restrict__ row_idx,
                                                               u32 n, const T* __restrict__ grads,
                                                               u32 units, u32 lp_full, u32 P) {
    const u32 lane = threadIdx.x & 63u;
    const u32 col0 = blockIdx.y * 64u;
    const u32 lp = (units - col0) < 64u ? (units - col0) : 64u;
    const u32 g = lane / lp_full;
    const u32 c = lane - g * lp_full;
    if (!(g < P && c < lp)) return;
    const u64 wave = ((u64)blockIdx.x * BLOCK + threadIdx.x) >> 6;
    const u64 nwaves = ((u64)gridDim.x * BLOCK) >> 6;
    for (u64 i = wave * P + g; i < n; i += nwaves * P) {
        u32 s = row_idx[i];
        if (s == SLOT_NONE) continue;
        T gv = grads[i * units + col0 + c];
        finalize<T>(t, s, col0 + c, units, gv);
    }
}

// ---- whole-value writes, record packing -------------------------------------------------------
__global__ __launch_bounds__(BLOCK) void write_values_kernel(TableDev t,
                                                              const u32* __restrict__ slot_idx,
                                                              u64 total, const float* __restrict__ values,
                                                              u64 m64) {
    for (u64 q = (u64)blockIdx.x * BLOCK + threadIdx.x; q < total; q += (u64)gridDim.x * BLOCK) {
        u64 i = div_big(q, m64, t.vf);
        u32 f = (u32)(q - i * t.vf);
        u32 s = slot_idx[i];
        if (s == SLOT_NONE) continue;
        u32 row = reinterpret_cast<const u32*>(&t.slots[s])[2];
        if (row >= t.max_rows) continue;
        t.rows[(u64)row * t.stride_f + f] = values[q];
    }
}

__global__ __launch_bounds__(BLOCK) void pack_records_kernel(TableDev t, u32 first_row, u64 total,
                                                              u32* __restrict__ rec, u32 rec_dw,
                                                              u64 m64) {
    const u32* rows = reinterpret_cast<const u32*>(t.rows);
    const u32* rk = reinterpret_cast<const u32*>(t.row_keys);
    for (u64 q = (u64)blockIdx.x * BLOCK + threadIdx.x; q < total; q += (u64)gridDim.x * BLOCK) {
        u64 r = div_big(q, m64, rec_dw);
        u32 off = (u32)(q - r * rec_dw);
        u64 row = first_row + r;
        rec[q] = off < 2 ? rk[row * 2 + off] : rows[row * t.stride_f + (off - 2)];
    }
}

__global__ __launch_bounds__(BLOCK) void pack_rows_kernel(TableDev t, const u32* __restrict__ row_list,
                                                           u64 total, u32* __restrict__ rec, u32 rec_dw,
                                                           u64 m64) {
    const u32* rows = reinterpret_cast<const u32*>(t.rows);
    const u32* rk = reinterpret_cast<const u32*>(t.row_keys);
    for (u64 q = (u64)blockIdx.x * BLOCK + threadIdx.x; q < total; q += (u64)gridDim.x * BLOCK) {
        u64 r = div_big(q, m64, rec_dw);
        u32 off = (u32)(q - r * rec_dw);
        u64 row = row_list[r];
        rec[q] = off < 2 ? rk[row * 2 + off] : rows[row * t.stride_f + (off - 2)];
        if (off == 0 && t.dirty) t.dirty[row] = 0;
    }
}

__global__ __launch_bounds__(BLOCK) void unpack_records_kernel(const u32* __restrict__ rec, u64 total,
                                                                u32 stride_dw, u32 fpr, u32* keys,
                                                                float* values, u64 m64) {
    const u32 used = fpr + 2;
    for (u64 q = (u64)blockIdx.x * BLOCK + threadIdx.x; q < total; q += (u64)gridDim.x * BLOCK) {
        u64 r = div_big(q, m64, used);
        u32 off = (u32)(q - r * used);
        u32 v = rec[r * stride_dw + off];
        if (off < 2)
            keys[r * 2 + off] = v;
        else
            reinterpret_cast<u32*>(values)[r * fpr + (off - 2)] = v;
    }
}

// distance, in buckets, between a stored key's home bucket and the bucket that holds it: four lanes
// per key walk the chain, the counts are kept per workgroup in LDS and added to `hist` once per
// workgroup and bin (additions to one address from all over the device are resolved one by one).
__global__ __launch_bounds__(BLOCK) void probe_hist_kernel(TableDev t, u32 n_rows,
                                                            unsigned long long* hist) {
    __shared__ u32 h[16];
    __shared__ u32 hmax;
    if (threadIdx.x < 16) h[threadIdx.x] = 0;
    if (threadIdx.x == 16) hmax = 0;
    __syncthreads();
    const u32 lane = threadIdx.x & 63u;
    const u32 grp = lane >> 2, sub = lane & 3u;
    const u64 wave = ((u64)blockIdx.x * BLOCK + threadIdx.x) >> 6;
    const u64 nwaves = ((u64)gridDim.x * BLOCK) >> 6;
    for (u64 base = wave * KEYS_PER_ROUND; base < n_rows; base += nwaves * KEYS_PER_ROUND) {
        const u64 r = base + grp;
        const u64 key = r < n_rows ? t.row_keys[r] : KEY_EMPTY;
        const bool active = key < KEY_DELETED;
        const Found f = probe_find(t, key, active, grp, sub);
        if (active && sub == 0 && f.slot != SLOT_NONE) {
            const u32 dist = ((f.slot >> 2) - ((u32)hash64(key) & t.bucket_mask)) & t.bucket_mask;
            atomicAdd(&h[dist < 15u ? dist : 15u], 1u);
            atomicMax(&hmax, dist);
        }
    }
    __syncthreads();
    if (threadIdx.x < 16 && h[threadIdx.x]) atomicAdd(&hist[threadIdx.x], (unsigned long long)h[threadIdx.x]);
    if (threadIdx.x == 16 && hmax) atomicMax(&hist[16], (unsigned long long)hmax);
}

inline u32 grid_for(u64 work_items, u32 per_block, u32 cap) {
    u64 b = (work_items + per_block - 1) / per_block;
    if (b < 1) b = 1;
    if (b > cap) b = cap;
    return (u32)b;
}

inline bool vec4_ok(const TableDev& t, const void* a, const void* b = nullptr) {
    return (t.dim % 4 == 0) && ((reinterpret_cast<uintptr_t>(a) & 15u) == 0) &&
           ((reinterpret_cast<uintptr_t>(b) & 15u) == 0);
}

}  // namespace

// ---- launchers -----------------------------------------------------------------------------
hipError_t launch_fill_u32(u32* p, size_t n, u32 v, hipStream_t s) {
    if (n == 0) return hipSuccess;
    fill_u32_kernel<<<grid_for(n, BLOCK, 65536), BLOCK, 0, s>>>(p, n, v);
    return hipGetLastError();
}

hipError_t launch_pull(const TableDev& t, const u64* keys, size_t n, float* out, uint8_t* hit, u32* handles,
                       hipStream_t s) {
    if (n == 0) return hipSuccess;
    const u32 grid = grid_for(n, KEYS_PER_ROUND * (BLOCK / 64), 16384);
    if (vec4_ok(t, out)) {
        u32 units = t.dim / 4;
        pull_kernel<float4><<<grid, BLOCK, 0, s>>>(t, keys, (u32)n, reinterpret_cast<float4*>(out),
                                                   hit, handles, units, t.stride_f / 4, magic32(units));
    } else {
        pull_kernel<float><<<grid, BLOCK, 0, s>>>(t, keys, (u32)n, out, hit, handles, t.dim, t.stride_f,
                                                  magic32(t.dim));
    }
    return hipGetLastError();
}

hipError_t launch_gather_slots(const TableDev& t, const u64* keys, const u32* slot_idx, size_t n, float* out,
                               uint8_t* hit, u32* handles, hipStream_t s) {
    if (n == 0) return hipSuccess;
    const u32 grid = grid_for(n, KEYS_PER_ROUND * (BLOCK / 64), 16384);
    if (vec4_ok(t, out)) {
        u32 units = t.dim / 4;
        gather_slots_kernel<float4><<<grid, BLOCK, 0, s>>>(t, keys, slot_idx, (u32)n,
                                                           reinterpret_cast<float4*>(out), hit, handles,
                                                           units, t.stride_f / 4, magic32(units));
    } else {
        gather_slots_kernel<float><<<grid, BLOCK, 0, s>>>(t, keys, slot_idx, (u32)n, out, hit, handles, t.dim,
                                                          t.stride_f, magic32(t.dim));
    }
    return hipGetLastError();
}

hipError_t launch_locate(const TableDev& t, const u64* keys, size_t n, u32* slot_out, u32* idx_out,
                         u32* row_out, u32* won_count, bool count_dups, hipStream_t s) {
    if (n == 0) return hipSuccess;
    const u32 grid = grid_for(n, KEYS_PER_ROUND * (BLOCK / 64), 16384);
    if (won_count)
        locate_kernel<true><<<grid, BLOCK, 0, s>>>(t, keys, (u32)n, slot_out, idx_out, row_out,
                                                   won_count, count_dups);
    else
        locate_kernel<false><<<grid, BLOCK, 0, s>>>(t, keys, (u32)n, slot_out, idx_out, row_out,
                                                    nullptr, count_dups);
    return hipGetLastError();
}

size_t assign_blocks(size_t n) { return (n + ASSIGN_KEYS - 1) / ASSIGN_KEYS; }

hipError_t launch_assign_rows(const TableDev& t, const u64* keys, size_t n, u32* slot_idx,
                              u32* row_out, const u32* won_count, u32* won_next, size_t won_words,
                              bool init_rows, hipStream_t s) {
    if (n == 0) return hipSuccess;
    const u32 n_blocks = (u32)assign_blocks(n);
    assign_rows_kernel<<<n_blocks, BLOCK, 0, s>>>(t, keys, (u32)n, slot_idx, row_out, won_count, won_next,
                                                  (u32)won_words, n_blocks, init_rows);
    return hipGetLastError();
}

hipError_t launch_rollback(const TableDev& t, const u32* slot_idx, size_t n, u32 first_new_row,
                           hipStream_t s) {
    rollback_kernel<<<grid_for(n ? n : 1, BLOCK, 1u << 30), BLOCK, 0, s>>>(t, slot_idx, (u32)n,
                                                                           first_new_row);
    return hipGetLastError();
}

hipError_t launch_segreduce(const TableDev& t, const u32* sorted_row, const u32* sorted_idx, size_t n,
                            const float* grads, uint4* part_hdr, float* part_val, hipStream_t s) {
    if (n == 0) return hipSuccess;
    const bool v4 = vec4_ok(t, grads, part_val);
    const SegGeom g = seg_geometry(t.dim, v4 ? 4 : 1, n);
    const u32 val_bytes = g.wch * g.lp * (v4 ? 16u : 4u);  // a multiple of 64
    const u32 arr_bytes = ((g.wch + 1) * 4u + 15u) & ~15u;
    const size_t lds = (size_t)(SEG_BLOCK / 64) * (val_bytes + 3 * arr_bytes);  // at most 57 KiB
    dim3 grid((g.n_chunks + SEG_BLOCK / 64 - 1) / (SEG_BLOCK / 64), g.col_blocks);
    if (v4)
        segreduce_kernel<float4><<<grid, SEG_BLOCK, lds, s>>>(
            t, sorted_row, sorted_idx, (u32)n, reinterpret_cast<const float4*>(grads), part_hdr,
            reinterpret_cast<float4*>(part_val), g.units, g.lp, g.p, g.wch, g.n_chunks, val_bytes,
            arr_bytes);
    else
        segreduce_kernel<float><<<grid, SEG_BLOCK, lds, s>>>(t, sorted_row, sorted_idx, (u32)n, grads,
                                                             part_hdr, part_val, g.units, g.lp, g.p,
                                                             g.wch, g.n_chunks, val_bytes, arr_bytes);
    return hipGetLastError();
}

// A window lies wholly inside a run only if the run entered it from the window before, so window 0
// never does: with fewer than two whole windows there is nothing for fixup_windows_kernel to add up,
// and fixup_kernel (which is told so by n_windows = 0) looks at no window. Windows are also left
// out while the longest chain they could shorten is short anyway: a run over all n_chunks chunks
// is found in n_chunks / 64 steps over the chunk headers and added by the P lane groups of one
// wavefront, four loads in flight each, in n_chunks / (4 P) steps; up to 8 such steps (about as
// long as the launch that would avoid them) fixup_windows_kernel costs more than it can save.
inline u32 window_count(u32 n_chunks, u32 P) {
    if (n_chunks < 2 * WINDOW || n_chunks <= 32u * P) return 0u;
    return (n_chunks + WINDOW - 1) / WINDOW;
}

hipError_t launch_fixup_windows(const TableDev& t, size_t n, const float* grads, const uint4* part_hdr,
                                const float* part_val, u32* win_row, float* win_val, hipStream_t s) {
    if (n == 0) return hipSuccess;
    const bool v4 = vec4_ok(t, grads, part_val) && vec4_ok(t, win_val);  // the layout launch_segreduce chose
    const SegGeom g = seg_geometry(t.dim, v4 ? 4 : 1, n);
    const u32 n_windows = window_count(g.n_chunks, g.p);
    if (n_windows == 0) return hipSuccess;
    dim3 grid((n_windows + BLOCK / 64 - 1) / (BLOCK / 64), g.col_blocks);  // a wavefront per window
    if (v4)
        fixup_windows_kernel<float4><<<grid, BLOCK, 0, s>>>(
            part_hdr, reinterpret_cast<const float4*>(part_val), win_row,
            reinterpret_cast<float4*>(win_val), g.units, g.lp, g.p, g.n_chunks, n_windows);
    else
        fixup_windows_kernel<float><<<grid, BLOCK, 0, s>>>(part_hdr, part_val, win_row, win_val,
                                                           g.units, g.lp, g.p, g.n_chunks, n_windows);
    return hipGetLastError();
}

hipError_t launch_fixup(const TableDev& t, size_t n, const float* grads, const uint4* part_hdr,
                        const float* part_val, const u32* win_row, const float* win_val,
                        hipStream_t s) {
    if (n == 0) return hipSuccess;
    const bool v4 = vec4_ok(t, grads, part_val) && vec4_ok(t, win_val);
    const SegGeom g = seg_geometry(t.dim, v4 ? 4 : 1, n);
    if (g.n_chunks <= 1) return hipSuccess;  // no border, no run across one
    const u32 n_windows = window_count(g.n_chunks, g.p);
    dim3 grid((g.n_chunks + BLOCK / 64 - 1) / (BLOCK / 64), g.col_blocks);  // a wavefront per chunk
    if (v4)
        fixup_kernel<float4><<<grid, BLOCK, 0, s>>>(
            t, part_hdr, reinterpret_cast<const float4*>(part_val), win_row,
            reinterpret_cast<const float4*>(win_val), g.units, g.lp, g.p, g.n_chunks, n_windows);
    else
        fixup_kernel<float><<<grid, BLOCK, 0, s>>>(t, part_hdr, part_val, win_row, win_val, g.units,
                                                   g.lp, g.p, g.n_chunks, n_windows);
    return hipGetLastError();
}

// One workgroup takes its keys 256 at a time, so its time grows with the batch where the chain of
// kernels spreads over the device: the one launch wins up to about 512 keys (256 keys: 15 µs
// against 29, 512: 25 against 30, 1024: 55 against 30).
size_t push_small_max() { return SMALL_PUSH / 2; }

hipError_t launch_push_small(const TableDev& t, const u64* keys, const float* grads, size_t n, bool insert,
                             hipStream_t s) {
    if (n == 0) return hipSuccess;
    if (n > SMALL_PUSH) return hipErrorInvalidValue;
    if (vec4_ok(t, grads))
        push_small_kernel<float4><<<1, SMALL_PUSH, 0, s>>>(t, keys, reinterpret_cast<const float4*>(grads),
                                                          (u32)n, insert ? 1 : 0, t.dim / 4);
    else
        push_small_kernel<float><<<1, SMALL_PUSH, 0, s>>>(t, keys, grads, (u32)n, insert ? 1 : 0, t.dim);
    return hipGetLastError();
}

hipError_t launch_update_unique(const TableDev& t, const u32* row_idx, size_t n, const float* grads,
                                hipStream_t s) {
    if (n == 0) return hipSuccess;
    const bool v4 = vec4_ok(t, grads);
    const SegGeom g = seg_geometry(t.dim, v4 ? 4 : 1, n);
    dim3 grid(grid_for(n, g.p * (BLOCK / 64), 16384), g.col_blocks);
    if (v4)
        update_unique_kernel<float4><<<grid, BLOCK, 0, s>>>(
            t, row_idx, (u32)n, reinterpret_cast<const float4*>(grads), g.units, g.lp, g.p);
    else
        update_unique_kernel<float><<<grid, BLOCK, 0, s>>>(t, row_idx, (u32)n, grads, g.units, g.lp,
                                                           g.p);
    return hipGetLastError();
}

hipError_t launch_write_values(const TableDev& t, const u32* slot_idx, size_t n, const float* values,
                               hipStream_t s) {
    if (n == 0) return hipSuccess;
    const u64 total = (u64)n * t.vf;
    write_values_kernel<<<grid_for(total, BLOCK * 4, 65536), BLOCK, 0, s>>>(t, slot_idx, total,
                                                                            values, magic64(t.vf));
    return hipGetLastError();
}

hipError_t launch_pack_records(const TableDev& t, u32 first_row, size_t n, u32* records,
                               hipStream_t s) {
    if (n == 0) return hipSuccess;
    const u32 rec_dw = t.vf + 2;
    const u64 total = (u64)n * rec_dw;
    pack_records_kernel<<<grid_for(total, BLOCK * 4, 65536), BLOCK, 0, s>>>(
        t, first_row, total, records, rec_dw, magic64(rec_dw));
    return hipGetLastError();
}

hipError_t launch_pack_rows(const TableDev& t, const u32* row_list, size_t n, u32* records, hipStream_t s) {
    if (n == 0) return hipSuccess;
    const u32 rec_dw = t.vf + 2;
    const u64 total = (u64)n * rec_dw;
    pack_rows_kernel<<<grid_for(total, BLOCK * 4, 65536), BLOCK, 0, s>>>(t, row_list, total, records, rec_dw,
                                                                        magic64(rec_dw));
    return hipGetLastError();
}

hipError_t launch_unpack_records(const u32* records, size_t n, u32 stride_dw, u32 floats_per_rec,
                                 u64* keys, float* values, hipStream_t s) {
    if (n == 0) return hipSuccess;
    const u32 used = floats_per_rec + 2;
    const u64 total = (u64)n * used;
    unpack_records_kernel<<<grid_for(total, BLOCK * 4, 65536), BLOCK, 0, s>>>(
        records, total, stride_dw, floats_per_rec, reinterpret_cast<u32*>(keys), values,
        magic64(used));
    return hipGetLastError();
}

hipError_t launch_probe_hist(const TableDev& t, u32 n_rows, unsigned long long* hist,
                             hipStream_t s) {
    if (n_rows == 0) return hipSuccess;
    probe_hist_kernel<<<grid_for(n_rows, KEYS_PER_ROUND * (BLOCK / 64) * 8, 16384), BLOCK, 0, s>>>(t, n_rows, hist);
    return hipGetLastError();
}

}  // namespace pshbm
