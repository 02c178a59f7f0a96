// Whole-table kernels: for-each with a predicate and a count / column-sum reduction, erase of the
// rows a predicate or a key list selects, and the rebuild of the hash array.
//
// Erasing keeps the row slab dense. With n rows of which E die, the n' = n - E survivors must end
// in rows [0, n'): every dead row below n' (a hole) receives a live row from [n', n) (a mover).
// A prefix count of the dead flags gives both lists without sorting: the h-th hole is the dead row
// with h dead rows before it, and it is paired with the live row that has h live rows after it.
// The slot of an erased key keeps a marker (KEY_DELETED) so that probe chains through it stay
// intact; markers are dropped when the hash array is rebuilt from the stored keys.
#include "../../include/pshbm.h"
#include "probe.h"
#include "table.h"

namespace pshbm {

namespace {

__device__ __forceinline__ bool cmp_f(float v, int32_t cmp, float f) {
    switch (cmp) {
        case PSHBM_CMP_LT: return v < f;
        case PSHBM_CMP_LE: return v <= f;
        case PSHBM_CMP_GT: return v > f;
        case PSHBM_CMP_GE: return v >= f;
        case PSHBM_CMP_EQ: return v == f;
        case PSHBM_CMP_NE: return v != f;
    }
    return false;
}

__device__ __forceinline__ bool cmp_u(u64 k, const pshbm_term& t) {
    switch (t.cmp) {
        case PSHBM_CMP_LT: return k < t.u;
        case PSHBM_CMP_LE: return k <= t.u;
        case PSHBM_CMP_GT: return k > t.u;
        case PSHBM_CMP_GE: return k >= t.u;
        case PSHBM_CMP_EQ: return k == t.u;
        case PSHBM_CMP_NE: return k != t.u;
        case PSHBM_CMP_MOD_EQ: return t.u != 0 && k % t.u == t.u2;
        case PSHBM_CMP_PART_EQ: return (u64)jump_partition(k, (int32_t)t.u) == t.u2;
        case PSHBM_CMP_PART_NE: return (u64)jump_partition(k, (int32_t)t.u) != t.u2;
    }
    return false;
}

__device__ __forceinline__ bool eval_pred(const pshbm_predicate& p, u64 key, const float* row) {
    bool ok = true;
    for (u32 i = 0; i < p.n_terms; ++i) {
        const pshbm_term& t = p.term[i];
        ok = ok && (t.column < 0 ? cmp_u(key, t) : cmp_f(row[t.column], t.cmp, t.f));
    }
    return ok;
}

// ---- for-each ------------------------------------------------------------------------------
// A workgroup of 256 threads = G groups of lp lanes (lp = columns handled at once); the workgroups
// take spans of G * FE_UNROLL consecutive rows in turn, group g every G-th row of a span, and lane c
// adds up column c of the rows that satisfy the predicate. The G sums of a column are then added in group order, and
// the per-workgroup results in workgroup order by for_each_final_kernel: a fixed order throughout.
// partial: [gridDim.x][vf + 1] doubles, the last one the count.
constexpr u32 FE_UNROLL = 8;
__global__ __launch_bounds__(BLOCK) void for_each_kernel(TableDev t, u32 n_rows, pshbm_predicate pred,
                                                          double* __restrict__ partial, u32 lp,
                                                          u32 G) {
    __shared__ double sh[BLOCK];
    __shared__ unsigned long long cnts[BLOCK];
    __shared__ uint8_t okf[BLOCK * FE_UNROLL];
    const u32 tid = threadIdx.x;
    const u32 g = tid / lp, cl = tid - g * lp;
    const u32 c = blockIdx.y * 256u + cl;
    const bool has_pred = pred.n_terms != 0;
    const u32 span = G * FE_UNROLL;  // consecutive rows the workgroup reads per step
    double acc = 0.0;
    unsigned long long cnt = 0;
    for (u64 s0 = (u64)blockIdx.x * span; s0 < n_rows; s0 += (u64)gridDim.x * span) {
        if (has_pred) {  // once per row, a thread per row; the flags go through LDS
            __syncthreads();
            for (u32 x = tid; x < span; x += BLOCK) {
                const u64 r = s0 + x;
                okf[x] = r < n_rows && eval_pred(pred, t.row_keys[r], t.rows + r * t.stride_f) ? 1 : 0;
            }
            __syncthreads();
        }
        if (g < G) {
            // FE_UNROLL rows per step, their loads issued together; a group adds its rows in
            // ascending order
            float v[FE_UNROLL];
            bool ok[FE_UNROLL];
#pragma unroll
            for (u32 k = 0; k < FE_UNROLL; ++k) {
                const u32 x = k * G + g;
                const u64 r = s0 + x;
                ok[k] = r < n_rows;
                v[k] = 0.0f;
                if (ok[k] && c < t.vf) v[k] = t.rows[r * t.stride_f + c];
            }
            if (has_pred) {
#pragma unroll
                for (u32 k = 0; k < FE_UNROLL; ++k) ok[k] = ok[k] && okf[k * G + g] != 0;
            }
#pragma unroll
            for (u32 k = 0; k < FE_UNROLL; ++k)
                if (ok[k]) {
                    acc += (double)v[k];
                    ++cnt;
                }
        }
    }
    sh[tid] = acc;
    cnts[tid] = cnt;
    __syncthreads();
    if (g == 0 && c < t.vf) {
        double s = 0.0;
        for (u32 x = 0; x < G; ++x) s += sh[x * lp + cl];
        partial[(u64)blockIdx.x * (t.vf + 1) + c] = s;
    }
    if (tid == 0 && blockIdx.y == 0) {
        unsigned long long s = 0;
        for (u32 x = 0; x < G; ++x) s += cnts[x * lp];
        partial[(u64)blockIdx.x * (t.vf + 1) + t.vf] = (double)s;  // exact below 2^53
    }
}

// Workgroup c adds up column c (c = vf: the count) of the per-workgroup results: thread x takes
// every BLOCK-th of them in ascending order, then the BLOCK sums are added in thread order.
__global__ __launch_bounds__(BLOCK) void for_each_final_kernel(const double* __restrict__ partial,
                                                                u32 n_blocks, u32 vf,
                                                                double* __restrict__ out) {
    __shared__ double sh[BLOCK];
    const u32 c = blockIdx.x;
    double s = 0.0;
    for (u32 b = threadIdx.x; b < n_blocks; b += BLOCK) s += partial[(u64)b * (vf + 1) + c];
    sh[threadIdx.x] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        double tot = 0.0;
        for (u32 x = 0; x < BLOCK; ++x) tot += sh[x];
        out[c] = tot;
    }
}

// Writing for-each, in the layout of for_each_kernel: the workgroups take spans of G * FE_UNROLL
// consecutive rows in turn; a thread per row evaluates the predicate on the row as it is before
// the rewrite (flags through LDS, the mark of a selected row is set here), then group g rewrites
// every G-th row of the span, lane c the columns c, c + 256, ... that `what` names.
// partial: the selected rows of every workgroup, added up in a fixed order afterwards.
__global__ __launch_bounds__(BLOCK) void for_each_write_kernel(TableDev t, u32 n_rows, pshbm_predicate pred,
                                                                pshbm_update what,
                                                                double* __restrict__ partial, u32 lp,
                                                                u32 G) {
    __shared__ u32 wsum[BLOCK / 64];
    __shared__ uint8_t okf[BLOCK * FE_UNROLL];
    const u32 tid = threadIdx.x;
    const u32 g = tid / lp, cl = tid - g * lp;
    const bool has_pred = pred.n_terms != 0;
    const u32 c_end = what.first_column + what.n_columns;
    const u32 span = G * FE_UNROLL;
    u32 mine = 0;
    for (u64 s0 = (u64)blockIdx.x * span; s0 < n_rows; s0 += (u64)gridDim.x * span) {
        __syncthreads();
        for (u32 x = tid; x < span; x += BLOCK) {
            const u64 r = s0 + x;
            const bool ok = r < n_rows &&
                            (!has_pred || eval_pred(pred, t.row_keys[r], t.rows + r * t.stride_f));
            okf[x] = ok ? 1 : 0;
            if (ok) {
                ++mine;
                if (t.dirty) t.dirty[r] = 1;
            }
        }
        __syncthreads();
        if (g >= G) continue;
        for (u32 c = cl; c < c_end; c += 256u) {
            if (c < what.first_column) continue;
            float v[FE_UNROLL];
            bool ok[FE_UNROLL];
#pragma unroll
            for (u32 k = 0; k < FE_UNROLL; ++k) {
                const u32 x = k * G + g;
                ok[k] = s0 + x < n_rows && okf[x] != 0;
                v[k] = 0.0f;
                if (ok[k]) v[k] = t.rows[(s0 + x) * t.stride_f + c];
            }
#pragma unroll
            for (u32 k = 0; k < FE_UNROLL; ++k) {
                if (!ok[k]) continue;
                float out;
                if (what.op == PSHBM_UPD_AFFINE) {
                    const float p = what.a * v[k];
                    out = p + what.b;
                } else {
                    out = fminf(fmaxf(v[k], what.a), what.b);
                }
                t.rows[(s0 + k * G + g) * t.stride_f + c] = out;
            }
        }
    }
    for (u32 off = 32; off >= 1; off >>= 1) mine += __shfl_down(mine, off);
    if ((tid & 63u) == 0) wsum[tid >> 6] = mine;
    __syncthreads();
    if (tid == 0) {
        u32 s = 0;
        for (u32 x = 0; x < BLOCK / 64; ++x) s += wsum[x];
        partial[blockIdx.x] = (double)s;
    }
}

__global__ __launch_bounds__(BLOCK) void sum_partials_kernel(const double* __restrict__ partial, u32 n,
                                                              double* __restrict__ out) {
    __shared__ double sh[BLOCK];
    double s = 0.0;
    for (u32 b = threadIdx.x; b < n; b += BLOCK) s += partial[b];
    sh[threadIdx.x] = s;
    __syncthreads();
    if (threadIdx.x == 0) {
        double tot = 0.0;
        for (u32 x = 0; x < BLOCK; ++x) tot += sh[x];
        out[0] = tot;
    }
}

// ---- erase ---------------------------------------------------------------------------------
__global__ __launch_bounds__(BLOCK) void mark_pred_kernel(TableDev t, u32 n_rows, pshbm_predicate pred,
                                                           uint8_t* __restrict__ dead) {
    const u64 r = (u64)blockIdx.x * BLOCK + threadIdx.x;
    if (r >= n_rows) return;
    dead[r] = eval_pred(pred, t.row_keys[r], t.rows + r * t.stride_f) ? 1 : 0;
}

__global__ __launch_bounds__(BLOCK) void mark_rows_kernel(const u32* __restrict__ rows, u32 n,
                                                           u32 n_rows, uint8_t* __restrict__ dead) {
    const u64 i = (u64)blockIdx.x * BLOCK + threadIdx.x;
    if (i >= n) return;
    const u32 r = rows[i];
    if (r < n_rows) dead[r] = 1;  // repeats of a key write the same byte
}

constexpr u32 ER_BLOCK = 1024, ER_ITEMS = 4, ER_TILE = ER_BLOCK * ER_ITEMS;

// dead rows of every tile of 4096 rows
__global__ __launch_bounds__(ER_BLOCK) void erase_count_kernel(const uint8_t* __restrict__ dead,
                                                               u32 n_rows, u32* __restrict__ tile_cnt) {
    __shared__ u32 wsum[ER_BLOCK / 64];
    const u32 tid = threadIdx.x;
    const u64 base = (u64)blockIdx.x * ER_TILE + (u64)tid * ER_ITEMS;
    u32 c = 0;
#pragma unroll
    for (u32 j = 0; j < ER_ITEMS; ++j)
        if (base + j < n_rows) c += dead[base + j];
    for (u32 off = 32; off >= 1; off >>= 1) c += __shfl_down(c, off);
    if ((tid & 63u) == 0) wsum[tid >> 6] = c;
    __syncthreads();
    if (tid == 0) {
        u32 s = 0;
        for (u32 x = 0; x < ER_BLOCK / 64; ++x) s += wsum[x];
        tile_cnt[blockIdx.x] = s;
    }
}

// One workgroup: tile_cnt becomes its exclusive prefix; info = {erased, rows left}; the row count
// of the table is set to the rows left.
__global__ __launch_bounds__(ER_BLOCK) void erase_scan_kernel(TableDev t, u32* __restrict__ tile_cnt,
                                                              u32 n_tiles, u32 n_rows,
                                                              u32* __restrict__ info, int set_row_count) {
    __shared__ u32 wsum[ER_BLOCK / 64];
    __shared__ u32 carry;
    const u32 tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    if (tid == 0) carry = 0;
    __syncthreads();
    for (u32 b0 = 0; b0 < n_tiles; b0 += ER_BLOCK) {
        const u32 i = b0 + tid;
        const u32 v = i < n_tiles ? tile_cnt[i] : 0u;
        u32 incl = v;
        for (u32 off = 1; off < 64; off <<= 1) {
            const u32 o = __shfl_up(incl, off);
            if (lane >= off) incl += o;
        }
        if (lane == 63) wsum[w] = incl;
        __syncthreads();
        u32 before = carry;
        for (u32 x = 0; x < w; ++x) before += wsum[x];
        if (i < n_tiles) tile_cnt[i] = before + incl - v;
        __syncthreads();
        if (tid == ER_BLOCK - 1) carry = before + incl;
        __syncthreads();
    }
    if (tid == 0) {
        info[0] = carry;
        info[1] = n_rows - carry;
        info[2] = 0;  // holes; set by erase_lists_kernel when there are any
        if (set_row_count) t.counters[CNT_ROWS] = n_rows - carry;
    }
}

// dead_list: every dead row, ascending. hole_list: the dead rows below n', ascending. mover_list:
// the live rows from n' on, descending. info[2] = number of holes.
__global__ __launch_bounds__(ER_BLOCK) void erase_lists_kernel(const uint8_t* __restrict__ dead,
                                                               u32 n_rows, const u32* __restrict__ tile_off,
                                                               u32* __restrict__ info,
                                                               u32* __restrict__ dead_list,
                                                               u32* __restrict__ hole_list,
                                                               u32* __restrict__ mover_list) {
    __shared__ u32 wsum[ER_BLOCK / 64];
    const u32 tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    const u32 erased = info[0], left = info[1];
    const u64 base = (u64)blockIdx.x * ER_TILE + (u64)tid * ER_ITEMS;
    u32 d[ER_ITEMS], c = 0;
#pragma unroll
    for (u32 j = 0; j < ER_ITEMS; ++j) {
        d[j] = base + j < n_rows ? dead[base + j] : 0u;
        c += d[j];
    }
    u32 incl = c;
    for (u32 off = 1; off < 64; off <<= 1) {
        const u32 o = __shfl_up(incl, off);
        if (lane >= off) incl += o;
    }
    if (lane == 63) wsum[w] = incl;
    __syncthreads();
    u32 before = tile_off[blockIdx.x] + incl - c;  // dead rows before this thread's first row
    for (u32 x = 0; x < w; ++x) before += wsum[x];
#pragma unroll
    for (u32 j = 0; j < ER_ITEMS; ++j) {
        const u64 r = base + j;
        if (r >= n_rows) break;
        if (r == left) info[2] = before;  // dead rows below n' = holes
        if (d[j]) {
            dead_list[before] = (u32)r;
            if (r < left) hole_list[before] = (u32)r;
            ++before;
        } else if (r >= left) {
            // live rows after r = rows after r - dead rows after r
            mover_list[(n_rows - 1 - (u32)r) - (erased - before)] = (u32)r;
        }
    }
}

// flagged rows, ascending (the prefix of the flags is in tile_off)
__global__ __launch_bounds__(ER_BLOCK) void flag_list_kernel(const uint8_t* __restrict__ flags, u32 n_rows,
                                                             const u32* __restrict__ tile_off,
                                                             u32* __restrict__ list) {
    __shared__ u32 wsum[ER_BLOCK / 64];
    const u32 tid = threadIdx.x, lane = tid & 63u, w = tid >> 6;
    const u64 base = (u64)blockIdx.x * ER_TILE + (u64)tid * ER_ITEMS;
    u32 d[ER_ITEMS], c = 0;
#pragma unroll
    for (u32 j = 0; j < ER_ITEMS; ++j) {
        d[j] = base + j < n_rows ? flags[base + j] : 0u;
        c += d[j];
    }
    u32 incl = c;
    for (u32 off = 1; off < 64; off <<= 1) {
        const u32 o = __shfl_up(incl, off);
        if (lane >= off) incl += o;
    }
    if (lane == 63) wsum[w] = incl;
    __syncthreads();
    u32 before = tile_off[blockIdx.x] + incl - c;
    for (u32 x = 0; x < w; ++x) before += wsum[x];
#pragma unroll
    for (u32 j = 0; j < ER_ITEMS; ++j)
        if (d[j]) list[before++] = (u32)(base + j);
}

// The slots of the erased keys become markers. 4 lanes per key.
__global__ __launch_bounds__(BLOCK) void erase_slots_kernel(TableDev t, const u32* __restrict__ dead_list,
                                                             const u32* __restrict__ info) {
    const u32 lane = threadIdx.x & 63u;
    const u32 grp = lane >> 2, sub = lane & 3u;
    const u32 n = info[0];
    const u64 wave = ((u64)blockIdx.x * BLOCK + threadIdx.x) >> 6;
    const u64 nwaves = ((u64)gridDim.x * BLOCK) >> 6;
    for (u64 base = wave * KEYS_PER_ROUND; base < n; base += nwaves * KEYS_PER_ROUND) {
        const u64 i = base + grp;
        const bool active = i < n;
        const u64 key = active ? t.row_keys[dead_list[i]] : KEY_EMPTY;
        const Found f = probe_find(t, key, active, grp, sub);
        if (active && sub == 0) {
            if (f.slot != SLOT_NONE)
                t.slots[f.slot] = make_uint4((u32)KEY_DELETED, (u32)(KEY_DELETED >> 32), ROW_NONE, 0u);
            if (t.dirty) t.dirty[dead_list[i]] = 0;  // rows past the row count carry no marks
        }
    }
}

// rows of the movers into the holes; units = 16-byte units per row
__global__ __launch_bounds__(BLOCK) void erase_move_kernel(TableDev t, const u32* __restrict__ hole_list,
                                                            const u32* __restrict__ mover_list,
                                                            const u32* __restrict__ info, u32 units) {
    const u64 total = (u64)info[2] * units;
    float4* rows = reinterpret_cast<float4*>(t.rows);
    for (u64 q = (u64)blockIdx.x * BLOCK + threadIdx.x; q < total; q += (u64)gridDim.x * BLOCK) {
        const u64 j = q / units;
        const u32 c = (u32)(q - j * units);
        const u32 dst = hole_list[j], src = mover_list[j];
        rows[(u64)dst * units + c] = rows[(u64)src * units + c];
        if (c == 0) {
            t.row_keys[dst] = t.row_keys[src];
            if (t.dirty) {  // the mark travels with the key
                t.dirty[dst] = t.dirty[src];
                t.dirty[src] = 0;
            }
        }
    }
}

// the slots of the moved keys point at their new rows
__global__ __launch_bounds__(BLOCK) void erase_repoint_kernel(TableDev t, const u32* __restrict__ hole_list,
                                                               const u32* __restrict__ mover_list,
                                                               const u32* __restrict__ info) {
    const u32 lane = threadIdx.x & 63u;
    const u32 grp = lane >> 2, sub = lane & 3u;
    const u32 n = info[2];
    const u64 wave = ((u64)blockIdx.x * BLOCK + threadIdx.x) >> 6;
    const u64 nwaves = ((u64)gridDim.x * BLOCK) >> 6;
    for (u64 base = wave * KEYS_PER_ROUND; base < n; base += nwaves * KEYS_PER_ROUND) {
        const u64 i = base + grp;
        const bool active = i < n;
        const u64 key = active ? t.row_keys[mover_list[i]] : KEY_EMPTY;
        const Found f = probe_find(t, key, active, grp, sub);
        if (active && sub == 0 && f.slot != SLOT_NONE)
            reinterpret_cast<u32*>(&t.slots[f.slot])[2] = hole_list[i];
    }
}

// Hash array rebuilt from row_keys: every key claims the first free slot from its home bucket on.
// The keys are distinct, so a slot that is taken belongs to another key.
__global__ __launch_bounds__(BLOCK) void reinsert_kernel(TableDev t, u32 n_rows) {
    const u32 lane = threadIdx.x & 63u;
    const u32 grp = lane >> 2, sub = lane & 3u;
    const u64 wave = ((u64)blockIdx.x * BLOCK + threadIdx.x) >> 6;
    const u64 nwaves = ((u64)gridDim.x * BLOCK) >> 6;
    for (u64 base = wave * KEYS_PER_ROUND; base < n_rows; base += nwaves * KEYS_PER_ROUND) {
        const u64 r = base + grp;
        const u64 key = r < n_rows ? t.row_keys[r] : KEY_EMPTY;
        bool done = !(r < n_rows);
        u32 b = (u32)hash64(key) & t.bucket_mask;
        u32 steps = 0;
        while (__ballot(!done)) {
            u64 skey = 0;
            if (!done)
                skey = __hip_atomic_load(reinterpret_cast<u64*>(&t.slots[(u64)b * 4 + sub]),
                                         __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            const bool empty = !done && skey == KEY_EMPTY;
            const u32 e4 = (u32)(__ballot(empty) >> (grp * 4)) & 0xFu;
            const u32 tgt = e4 ? (u32)__ffs((int)e4) - 1u : 0u;
            u64 old = 0;
            if (!done && e4 && sub == tgt)
                old = atomicCAS(reinterpret_cast<unsigned long long*>(&t.slots[(u64)b * 4 + tgt]),
                                (unsigned long long)KEY_EMPTY, (unsigned long long)key);
            const u64 oldb = shfl64(old, grp * 4 + tgt);
            if (!done) {
                if (e4) {
                    if (oldb == KEY_EMPTY) {
                        if (sub == tgt) reinterpret_cast<u32*>(&t.slots[(u64)b * 4 + tgt])[2] = (u32)r;
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
    }
}

inline u32 blocks_for(u64 items, u32 per_block, u32 cap) {
    u64 b = (items + per_block - 1) / per_block;
    if (b < 1) b = 1;
    if (b > cap) b = cap;
    return (u32)b;
}

constexpr u32 FE_BLOCKS_MAX = 2048;

u32 for_each_blocks(const TableDev& t, u32 n_rows, u32* lp_out, u32* g_out) {
    const u32 lp = t.vf < 256u ? t.vf : 256u;
    const u32 G = 256u / lp;
    *lp_out = lp;
    *g_out = G;
    return blocks_for(n_rows, G * 64u, FE_BLOCKS_MAX);
}

}  // namespace

size_t for_each_scratch_bytes(const TableDev& t) {
    return ((size_t)FE_BLOCKS_MAX + 1) * (t.vf + 1) * sizeof(double);
}

hipError_t launch_for_each(const TableDev& t, uint32_t n_rows, const pshbm_predicate& pred,
                           double* scratch, hipStream_t s) {
    u32 lp, G;
    const u32 n_blocks = for_each_blocks(t, n_rows, &lp, &G);
    double* partial = scratch + (t.vf + 1);
    dim3 grid(n_blocks, (t.vf + 255u) / 256u);
    for_each_kernel<<<grid, BLOCK, 0, s>>>(t, n_rows, pred, partial, lp, G);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    for_each_final_kernel<<<t.vf + 1, BLOCK, 0, s>>>(partial, n_blocks, t.vf, scratch);
    return hipGetLastError();
}

hipError_t launch_for_each_write(const TableDev& t, uint32_t n_rows, const pshbm_predicate& pred,
                                 const pshbm_update& what, double* scratch, hipStream_t s) {
    u32 lp, G;
    const u32 n_blocks = for_each_blocks(t, n_rows, &lp, &G);
    double* partial = scratch + (t.vf + 1);
    for_each_write_kernel<<<n_blocks, BLOCK, 0, s>>>(t, n_rows, pred, what, partial, lp, G);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    sum_partials_kernel<<<1, BLOCK, 0, s>>>(partial, n_blocks, scratch);
    return hipGetLastError();
}

hipError_t launch_mark_pred(const TableDev& t, uint32_t n_rows, const pshbm_predicate& pred,
                            uint8_t* dead, hipStream_t s) {
    if (n_rows == 0) return hipSuccess;
    mark_pred_kernel<<<blocks_for(n_rows, BLOCK, 1u << 30), BLOCK, 0, s>>>(t, n_rows, pred, dead);
    return hipGetLastError();
}

hipError_t launch_mark_rows(const uint32_t* rows, size_t n, uint32_t n_rows, uint8_t* dead,
                            hipStream_t s) {
    if (n == 0) return hipSuccess;
    mark_rows_kernel<<<blocks_for(n, BLOCK, 1u << 30), BLOCK, 0, s>>>(rows, (u32)n, n_rows, dead);
    return hipGetLastError();
}

size_t erase_tiles(uint32_t n_rows) { return ((size_t)n_rows + ER_TILE - 1) / ER_TILE; }

hipError_t launch_erase_count(const TableDev& t, uint32_t n_rows, const uint8_t* dead, uint32_t* tile_cnt,
                              uint32_t* info, hipStream_t s, bool set_row_count) {
    const u32 n_tiles = (u32)erase_tiles(n_rows);
    erase_count_kernel<<<n_tiles, ER_BLOCK, 0, s>>>(dead, n_rows, tile_cnt);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    erase_scan_kernel<<<1, ER_BLOCK, 0, s>>>(t, tile_cnt, n_tiles, n_rows, info, set_row_count ? 1 : 0);
    return hipGetLastError();
}

hipError_t launch_flag_list(uint32_t n_rows, const uint8_t* flags, const uint32_t* tile_off, uint32_t* list,
                            hipStream_t s) {
    if (n_rows == 0) return hipSuccess;
    flag_list_kernel<<<(u32)erase_tiles(n_rows), ER_BLOCK, 0, s>>>(flags, n_rows, tile_off, list);
    return hipGetLastError();
}

hipError_t launch_erase_apply(const TableDev& t, uint32_t n_rows, uint32_t erased, const uint8_t* dead,
                              const uint32_t* tile_off, uint32_t* info, uint32_t* lists, hipStream_t s) {
    u32* dead_list = lists;
    u32* hole_list = lists + erased;
    u32* mover_list = lists + 2 * (size_t)erased;
    erase_lists_kernel<<<(u32)erase_tiles(n_rows), ER_BLOCK, 0, s>>>(dead, n_rows, tile_off, info,
                                                                    dead_list, hole_list, mover_list);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return e;
    const u32 probe_grid = blocks_for(erased, KEYS_PER_ROUND * (BLOCK / 64), 16384);
    erase_slots_kernel<<<probe_grid, BLOCK, 0, s>>>(t, dead_list, info);
    if ((e = hipGetLastError()) != hipSuccess) return e;
    const u32 units = t.stride_f / 4;
    erase_move_kernel<<<blocks_for((u64)erased * units, BLOCK, 65536), BLOCK, 0, s>>>(t, hole_list,
                                                                                    mover_list, info, units);
    if ((e = hipGetLastError()) != hipSuccess) return e;
    erase_repoint_kernel<<<probe_grid, BLOCK, 0, s>>>(t, hole_list, mover_list, info);
    return hipGetLastError();
}

hipError_t launch_reinsert(const TableDev& t, uint32_t n_rows, hipStream_t s) {
    if (n_rows == 0) return hipSuccess;
    reinsert_kernel<<<blocks_for(n_rows, KEYS_PER_ROUND * (BLOCK / 64), 16384), BLOCK, 0, s>>>(t, n_rows);
    return hipGetLastError();
}

}  // namespace pshbm
