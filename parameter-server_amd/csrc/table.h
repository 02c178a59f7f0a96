// Device-side layout of one HBM-resident shard and the launch interface of its kernels.
//
// Hash array: `nbuckets` (a power of two) buckets of 4 slots; a slot is 16 bytes
// {uint64 key, uint32 row, uint32 aux}, so a bucket is one 64-byte line that four lanes read with
// one dwordx4 load each. A key lives in the first bucket, walking linearly from its home bucket,
// that had a free slot when it was inserted; buckets never lose keys while inserts run, so a
// lookup stops at the first bucket that still has an empty slot.
// Rows: dense slab `rows[row * stride_f]`, `vf` floats used per row (weights then optimizer
// state), numbered densely in batch order as keys are inserted and kept dense by erase (the last
// rows move into the holes); `row_keys[row]` is the key that owns the row, which makes Dump /
// iterate a linear walk of the slab.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/pshbm.h"

namespace pshbm {

constexpr uint64_t KEY_EMPTY = 0xFFFFFFFFFFFFFFFFull;
constexpr uint64_t KEY_DELETED = 0xFFFFFFFFFFFFFFFEull;
constexpr uint32_t ROW_NONE = 0xFFFFFFFFu;
constexpr uint32_t SLOT_NONE = 0xFFFFFFFFu;
// row of a key whose slot was claimed in the running operation, before rows are handed out
constexpr uint32_t ROW_PENDING = 0xFFFFFFFEu;

// indices into TableDev::counters
enum {
    CNT_ROWS = 0,      // rows handed out = keys stored
    CNT_OVERFLOW = 1,  // set when an insert found no row or no slot
    CNT_DUP = 2,       // keys that were already present (counted on request)
    CNT_ENTRY = 3,     // CNT_ROWS as it was when the current inserting operation began
    CNT_BADKEY = 4,    // reserved keys met in a batch (skipped)
    CNT_SORT_ERR = 5,  // a sort tile gave up waiting for its predecessor
    CNT_PART_ERR = 6,  // a partition of a push held more entries of one hash class than a pass takes
    CNT_ANY_NEW = 7,   // the partitioned push that is running has claimed a slot for a new key
    CNT_WORDS = 8
};

struct OptParams {
    int32_t kind;    // PSHBM_OPT_*
    int32_t states;  // blocks of dim floats after the weights: 0 SUM / SGD, 1 ADAGRAD, 2 FTRL, USER as user_opt.h says
    float lr, init_acc, alpha, beta, l1, l2;
    float init_range;  // weights of a new key: 0, or uniform in [-init_range, init_range) by init_weight()
};

struct TableDev {
    uint4* slots;        // nbuckets * 4
    float* rows;         // max_rows * stride_f
    uint64_t* row_keys;  // max_rows
    uint32_t* counters;  // CNT_WORDS
    uint8_t* dirty;      // max_rows bytes, or null: 1 = a push updated the row since the last take
    unsigned long long* pub;  // page-locked host word: {op_seq, rows} as the last inserting operation left them
    unsigned long long* part_stat;  // page-locked host word: {keys, entries} of the last partitioned push
    uint32_t bucket_mask;
    uint32_t max_rows;
    uint32_t dim;       // weights per key
    uint32_t vf;        // floats per value = dim * (1 + state blocks)
    uint32_t stride_f;  // floats between rows, multiple of 4
    uint32_t op_seq;    // number of the inserting operation this launch belongs to (set per launch)
    OptParams opt;
};

__host__ __device__ inline uint64_t hash64(uint64_t h) {
    h ^= h >> 33;
    h *= 0xff51afd7ed558ccdull;
    h ^= h >> 33;
    h *= 0xc4ceb9fe1a85ec53ull;
    h ^= h >> 33;
    return h;
}

// The partition of a key among n (1 .. 2^31-1): the shape of the reference's DefaultPartitioner<uint64_t>
// (pico-ps/common/Partitioner.h:43-61: jump_consistent_hash(murmur_hash(key), n)), with the published
// functions in the place of pico-core's: MurmurHash3's 64-bit finalizer and the jump consistent hash of
// Lamping and Veach (arXiv:1406.2294, the loop below is the paper's). The two floating-point operations
// are IEEE double division and multiplication on the host and on the device alike.
__host__ __device__ inline int32_t jump_partition(uint64_t key, int32_t n) {
    uint64_t k = hash64(key);
    int64_t b = -1, j = 0;
    while (j < n) {
        b = j;
        k = k * 2862933555777941757ull + 1;
        const double q = 2147483648.0 / (double)((k >> 33) + 1);
        j = (int64_t)((double)(b + 1) * q);
    }
    return (int32_t)b;
}

// Weight `col` of a key that is inserted, when the table draws initial weights: a pure function
// of key and column (24 bits of a hash, mapped to [-1, 1) exactly, times the range with one
// rounding), so that every path -- and the CPU restatement -- gives the key the same weights.
__host__ __device__ inline float init_weight(float range, uint64_t key, uint32_t col) {
    const uint64_t h = hash64(key ^ ((uint64_t)(col + 1u) * 0x9E3779B97F4A7C15ull));
    const float u = (float)(uint32_t)(h >> 40);
    const float x = u * 1.1920928955078125e-07f - 1.0f;
    return x * range;
}

// Segment-reduce geometry shared by the kernels and the host that sizes their scratch.
struct SegGeom {
    uint32_t units;       // row length in elements of the vector type (dim / vec)
    uint32_t col_blocks;  // ceil(units / 64)
    uint32_t lp;          // lanes per position in a full column block
    uint32_t p;           // positions per wave round
    uint32_t wch;         // positions per wave chunk
    uint32_t n_chunks;    // for a batch of n positions
};
constexpr uint32_t SEG_ROUNDS = 8;

inline SegGeom seg_geometry(uint32_t dim, uint32_t vec, uint64_t n) {
    SegGeom g;
    g.units = dim / vec;
    g.col_blocks = (g.units + 63) / 64;
    g.lp = g.units < 64 ? g.units : 64;
    g.p = 64 / g.lp;
    g.wch = g.p * SEG_ROUNDS;
    g.n_chunks = (uint32_t)((n + g.wch - 1) / g.wch);
    return g;
}

// ---- launchers (kernels.hip) ---------------------------------------------------------------
// All enqueue on `s` and return the hipError_t of the launch.

hipError_t launch_fill_u32(uint32_t* p, size_t n, uint32_t v, hipStream_t s);

// Fused probe + gather of pull without insertion. out is n x dim floats; hit may be null;
// handles (may be null): handles[i] = row of keys[i], or ROW_NONE.
hipError_t launch_pull(const TableDev& t, const uint64_t* keys, size_t n, float* out, uint8_t* hit,
                       uint32_t* handles, hipStream_t s);

// slot_out[i] = slot holding keys[i] or SLOT_NONE; idx_out[i] = i when idx_out is not null.
// won_count != null: claim a slot for each missing key (insert). The claiming occurrence has the
// top bit set in slot_out and is counted in won_count[i / 1024]; the launch also records the row
// count at entry (CNT_ENTRY). launch_assign_rows must follow: it gives the claimed slots dense row
// ids, fills row_keys, initialises the rows if asked, clears the top bits, publishes the new row
// count, and zeroes won_next (assign_blocks(n) words), the array the next operation counts into.
// count_dups: count keys that were found present or claimed by another lane into CNT_DUP.
// row_out (may be null): row_out[i] = row of keys[i], ROW_NONE if the key is not stored, or
// ROW_PENDING if its slot was claimed in this launch; launch_assign_rows fills in the rows of the
// claiming occurrences, and a later occurrence of such a key stays ROW_PENDING: its row is
// slots[slot_out[i]].z once launch_assign_rows has run (SortLateKeys does that lookup).
hipError_t launch_locate(const TableDev& t, const uint64_t* keys, size_t n, uint32_t* slot_out,
                         uint32_t* idx_out, uint32_t* row_out, uint32_t* won_count, bool count_dups,
                         hipStream_t s);
size_t assign_blocks(size_t n);
hipError_t launch_assign_rows(const TableDev& t, const uint64_t* keys, size_t n, uint32_t* slot_idx,
                              uint32_t* row_out, const uint32_t* won_count, uint32_t* won_next,
                              size_t won_words, bool init_rows, hipStream_t s);

// Gather through located slots (pull with insertion); hit = row existed when the pull began.
hipError_t launch_gather_slots(const TableDev& t, const uint64_t* keys, const uint32_t* slot_idx, size_t n, float* out,
                               uint8_t* hit, uint32_t* handles, hipStream_t s);

// Undo of a batch of claims: every located slot whose row is >= first_new_row (or unset) is
// emptied, the counters are restored.
hipError_t launch_rollback(const TableDev& t, const uint32_t* slot_idx, size_t n,
                           uint32_t first_new_row, hipStream_t s);

// Duplicate aggregation + update over (row, batch index) pairs sorted by row (ROW_NONE = key not
// stored, sorted last and skipped), in three launches: launch_segreduce
// sums runs of equal rows inside each wavefront's chunk and applies the complete ones;
// launch_fixup joins the runs that cross chunk borders. part_hdr: n_chunks uint4;
// part_val: n_chunks * 2 * dim floats.
hipError_t launch_segreduce(const TableDev& t, const uint32_t* sorted_row, const uint32_t* sorted_idx,
                            size_t n, const float* grads, uint4* part_hdr, float* part_val,
                            hipStream_t s);
// launch_fixup_windows first adds up every window of 64 chunks that lies wholly inside one run
// (win_row: n_chunks/64 + 1 words, win_val: as many rows of dim floats), so that launch_fixup can
// cross such a run a window at a time.
hipError_t launch_fixup_windows(const TableDev& t, size_t n, const float* grads, const uint4* part_hdr,
                                const float* part_val, uint32_t* win_row, float* win_val,
                                hipStream_t s);
hipError_t launch_fixup(const TableDev& t, size_t n, const float* grads, const uint4* part_hdr,
                        const float* part_val, const uint32_t* win_row, const float* win_val,
                        hipStream_t s);

// A whole push (probe and claim, rows for new keys, aggregation, update) of up to push_small_max()
// keys in one launch of one workgroup. The caller has made sure that the new keys fit.
size_t push_small_max();
hipError_t launch_push_small(const TableDev& t, const uint64_t* keys, const float* grads, size_t n,
                             bool insert, hipStream_t s);

// One optimizer step per located key, no aggregation (keys distinct); rows[i] = row of key i.
hipError_t launch_update_unique(const TableDev& t, const uint32_t* rows, size_t n,
                                const float* grads, hipStream_t s);

// rows[slot->row] = values[i] (whole value, vf floats).
hipError_t launch_write_values(const TableDev& t, const uint32_t* slot_idx, size_t n,
                               const float* values, hipStream_t s);

// records [first_row, first_row + n) of the slab as {key, vf floats} packed records.
hipError_t launch_pack_records(const TableDev& t, uint32_t first_row, size_t n, uint32_t* records,
                               hipStream_t s);
// the inverse split of packed records into a key array and a value matrix (n x floats_per_rec),
// record stride in dwords.
hipError_t launch_unpack_records(const uint32_t* records, size_t n, uint32_t stride_dw,
                                 uint32_t floats_per_rec, uint64_t* keys, float* values,
                                 hipStream_t s);

// probe-distance histogram over the stored keys: hist[0..15], hist[16] = max distance.
hipError_t launch_probe_hist(const TableDev& t, uint32_t n_rows, unsigned long long* hist,
                             hipStream_t s);

// ---- partitioned push (push_part.hip) ---------------------------------------------------------
// Aggregation and update of a batch of PART_MIN_KEYS .. PART_MAX_KEYS keys without a global sort:
// tiles of 4096 keys, partitions of about 1024 keys (ranges of home buckets). part_plan says whether a batch qualifies (and
// how it is cut); part_sizes gives the bytes of each scratch array for batches of up to n keys.
// (Below PART_MIN_KEYS one workgroup does the whole push in one launch; above PART_MAX_KEYS, and for
// a table so full that a batch may have to be undone, the sorted push takes over.)
constexpr size_t PART_MIN_KEYS = 513, PART_MAX_KEYS = 1u << 22;
struct PartPlan {
    uint32_t n, n_tiles, P, part_shift;
};
struct PartSizes {
    size_t stage, starts, pstart, psum, new_slot, new_count, ngrad, psize, order, resv;
};
struct PartBufs {
    uint4* stage;  // entries {key low, key high, reference, row handle}: a block per tile, grouped by partition
    uint32_t *starts, *pstart, *new_slot, *new_count;
    float *psum, *ngrad;
    uint32_t* psize;  // entries each partition held in the last push
    uint32_t* order;  // what each workgroup of the apply kernel should take: partitions, fullest first
    uint32_t* resv;   // per partition, zero between pushes: room reserved by the workgroups that share it
};
// entries_per_key: what the tiles of recent batches left per key (1 = no key repeats inside a tile);
// partitions are sized so that a pass of the apply kernel is well filled but rarely overflows.
bool part_plan(const TableDev& t, size_t n, double entries_per_key, PartPlan* plan);
PartSizes part_sizes(uint32_t dim, size_t n);
hipError_t part_init();  // once per device, before the first launch
// handles (may be null): the row of every key as an earlier pull of the same keys reported it
// (ROW_NONE where it found none); the apply kernel then looks up only the keys without one.
// verify: a handle counts only if row_keys[handle] is the key.
hipError_t launch_part_tile(const TableDev& t, const PartPlan& pl, const PartBufs& b, const uint64_t* keys,
                            const float* grads, const uint32_t* handles, hipStream_t s);
// use_order: workgroup x takes work item b.order[x] (left by an earlier push with the same plan: the
// partitions fullest first, the crowded ones shared by several workgroups); otherwise the partitions go
// round the XCDs in turn.
hipError_t launch_part_apply(const TableDev& t, const PartPlan& pl, const PartBufs& b, const float* grads, bool insert,
                             bool handles, bool verify, bool use_order, hipStream_t s);
// used_order: what the apply kernel was launched with. make_order: also rank the partitions by the
// entries the apply kernel found in them (b.psize) into b.order, and clear b.resv.
hipError_t launch_part_insert(const TableDev& t, const PartPlan& pl, const PartBufs& b, const float* grads,
                              bool used_order, bool make_order, hipStream_t s);
// Partitions from which an order pays: the apply kernel's workgroups then run in several rounds.
constexpr uint32_t PART_ORDER_MIN = 1024;
// Layout of PartBufs::order: the slots of a plan of P partitions (P + P / 8 of them), and at
// PART_ORDER_TAG the two words {P, bucket mask} of the plan it was made for.
constexpr uint32_t PART_MAX_PARTS = 4096;
constexpr uint32_t PART_ORDER_TAG = PART_MAX_PARTS + PART_MAX_PARTS / 8;
inline uint32_t part_order_slots(uint32_t P) { return P + P / 8; }
// Entries a pass of the apply kernel takes (0 = the default, 2048): a test hook that makes small
// batches go through the multi-pass path.
void part_set_pass_capacity(uint32_t entries);
// Smallest batch that takes the partitioned path (0 = the default, PART_MIN_KEYS): a test hook that
// sends mid-size batches through the sorted push.
void part_set_min_keys(size_t keys);

// ---- for-each / erase / rebuild (maint.hip) -------------------------------------------------
// Count and column sums of the rows that satisfy `pred`. scratch: for_each_scratch_bytes();
// the result is left in its first vf + 1 doubles (column sums, then the count).
size_t for_each_scratch_bytes(const TableDev& t);
hipError_t launch_for_each(const TableDev& t, uint32_t n_rows, const ::pshbm_predicate& pred,
                           double* scratch, hipStream_t s);
// Rewrites columns of the rows that satisfy `pred` (see pshbm_update); scratch as for
// launch_for_each, the count of rewritten rows is left in its first double.
hipError_t launch_for_each_write(const TableDev& t, uint32_t n_rows, const ::pshbm_predicate& pred,
                                 const ::pshbm_update& what, double* scratch, hipStream_t s);
// dead[r] = 1 where row r satisfies `pred`, else 0 / dead[rows[i]] = 1 for every rows[i] < n_rows.
hipError_t launch_mark_pred(const TableDev& t, uint32_t n_rows, const ::pshbm_predicate& pred,
                            uint8_t* dead, hipStream_t s);
hipError_t launch_mark_rows(const uint32_t* rows, size_t n, uint32_t n_rows, uint8_t* dead,
                            hipStream_t s);
// Erase of the flagged rows in two steps. launch_erase_count: tile_cnt (erase_tiles(n_rows) + 1
// words) becomes the prefix of the dead rows per tile of 4096 rows, info = {erased, rows left, -}
// and the table's row count becomes the rows left. launch_erase_apply (erased = info[0], read back
// by the host; lists: 3 * erased words): the erased keys' slots become markers, the surviving rows
// are packed into [0, rows left) and their slots follow them.
size_t erase_tiles(uint32_t n_rows);
hipError_t launch_erase_count(const TableDev& t, uint32_t n_rows, const uint8_t* dead, uint32_t* tile_cnt,
                              uint32_t* info, hipStream_t s, bool set_row_count = true);
// The flagged rows, ascending, after launch_erase_count(..., false): list holds info[0] words.
hipError_t launch_flag_list(uint32_t n_rows, const uint8_t* flags, const uint32_t* tile_off,
                            uint32_t* list, hipStream_t s);
// {key, value} records of the listed rows; clears their dirty marks.
hipError_t launch_pack_rows(const TableDev& t, const uint32_t* row_list, size_t n, uint32_t* records,
                            hipStream_t s);
hipError_t launch_erase_apply(const TableDev& t, uint32_t n_rows, uint32_t erased, const uint8_t* dead,
                              const uint32_t* tile_off, uint32_t* info, uint32_t* lists, hipStream_t s);
// Every row < n_rows claims a slot for its key in a hash array that the caller has emptied.
hipError_t launch_reinsert(const TableDev& t, uint32_t n_rows, hipStream_t s);

// ---- sort (sort.hip) -----------------------------------------------------------------------
// Stable radix sort of (key, value) pairs on the low `end_bit` bits (rounded up to whole digits of
// 8 to 10 bits: as few digit passes as 10-bit digits allow).
// Both buffer pairs are scratch: the sorted pairs end in (keys_b, vals_b) when *result_in_b, else
// in (keys_a, vals_a). *err_flag (device) is raised if a tile's bounded wait for its predecessor
// ran out, in which case the output is not sorted.
// `temp` starts with a head of sort_pairs_head_bytes() that must be zero before the first sort
// and is kept zeroed by the sorts themselves as long as `parity` alternates 0,1,0,1,...
size_t sort_pairs_temp_bytes(size_t n);
size_t sort_pairs_head_bytes();
// How many times a tile of a one-launch pass polls for a predecessor's counts before it gives up
// and raises the error flag (~0u = the default). 0 makes every waiting tile give up at once: the
// way a test reaches the failure path while every kernel still runs to its end.
void sort_set_spin_limit(uint32_t polls);
// The same sort step by step (sort_begin counts, then sort_pass places digit p = 0 .. passes-1,
// alternating between the two buffer pairs), for callers that time or interleave the launches.
// late (may be null): every keys[i] equal to late->marker is first replaced (for inputs of more
// than one tile in `keys` too) by late->table[late->index[i]].z.
struct SortLateKeys {
    uint32_t marker;
    const uint32_t* index;
    const uint4* table;
};
struct SortPlan {
    uint32_t n, n_tiles, bits;
    uint32_t passes;        // sort_pass calls to make
    uint32_t digit_passes;  // digit passes; all of them happen in one call when the input is one tile
    bool one_tile;          // up to 4096 pairs: one launch sorts them in LDS; sort_begin launches
                            // nothing, and the sort uses neither half of the head (`uses_head`)
    bool uses_head;         // the caller alternates `parity` only over the sorts that do
    bool lookback;          // otherwise: one launch per pass (up to 2^20 pairs) or three
    uint32_t* totals;
    uint32_t* status;
    size_t rows;
    SortLateKeys late;
};
hipError_t sort_begin(void* temp, size_t temp_bytes, unsigned parity, uint32_t* keys, size_t n,
                      unsigned end_bit, SortPlan* plan, hipStream_t s,
                      const SortLateKeys* late = nullptr);
hipError_t sort_pass(const SortPlan& plan, unsigned p, const uint32_t* kin, const uint32_t* vin,
                     uint32_t* kout, uint32_t* vout, uint32_t* err_flag, hipStream_t s);
hipError_t sort_pairs(void* temp, size_t temp_bytes, unsigned parity, uint32_t* keys_a,
                      uint32_t* keys_b, uint32_t* vals_a, uint32_t* vals_b, size_t n,
                      unsigned end_bit, bool* result_in_b, uint32_t* err_flag, hipStream_t s);

}  // namespace pshbm
