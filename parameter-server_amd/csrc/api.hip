// C ABI of the HBM sparse table (include/pshbm.h): host-side state, capacity accounting, stream
// ordering and staging around the kernels of kernels.hip / sort.hip.
#include "../../include/pshbm.h"

#include <algorithm>
#include <atomic>
#include <chrono>
#include <cstdarg>
#include <cstdio>
#include <cstring>
#include <deque>
#include <mutex>
#include <new>
#include <shared_mutex>
#include <string>
#include <thread>
#include <unordered_map>
#include <vector>

#include "table.h"
#include "user_opt.h"

using namespace pshbm;

namespace {

constexpr size_t BULK_CHUNK_BYTES = 32u << 20;  // staging granule of load / dump
constexpr uint32_t MAX_DIM = 16384;
constexpr size_t MAX_PUSH_BATCH = (1u << 30) - 1;  // the sort's tile counters hold 30 bits
constexpr size_t SMALL_HOST_BYTES = 1u << 20;       // host-pointer calls up to this size are staged

inline size_t round_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

struct DevBuf {
    void* p = nullptr;
    size_t bytes = 0;
};

// Scratch of one push: where the probe leaves slots, rows and batch indices, the sort's buffers, the
// partial sums of the segmented reduction. The table's own workspace grows with the batch; the
// entry point that must not allocate brings a fixed one.
struct Workspace {
    uint32_t *slot, *idx, *row, *srow, *sidx;
    void* sort;
    size_t sort_bytes;
    unsigned sort_parity;  // which half of the sort head is zero and will be used
    uint4* hdr;
    float* pval;
    uint32_t* wrow;
    float* wval;
    uint32_t *won_cur, *won_next;  // per-block winner counts: counted into / zeroed for the next operation
    size_t won_words;
    PartBufs part;    // scratch of the partitioned push, for batches of up to part_keys keys (0: none)
    size_t part_keys;
};

// Is [p, p + bytes) page-locked host memory that the runtime knows (hipHostMalloc,
// pshbm_host_alloc)? Then the copy engines can reach it and bulk transfers need no staging.
bool is_pinned_host(const void* p, size_t bytes) {
    if (!p || bytes == 0) return false;
    const void* ends[2] = {p, static_cast<const char*>(p) + bytes - 1};
    for (const void* q : ends) {
        hipPointerAttribute_t a{};
        if (hipPointerGetAttributes(&a, q) != hipSuccess) {
            (void)hipGetLastError();  // an ordinary pointer is not an error of the caller
            return false;
        }
        if (a.type != hipMemoryTypeHost) return false;
    }
    return true;
}

// memcpy between pageable memory and the staging buffers, split over a few threads: one thread
// moves about 10 GB/s, a third of what the link to the device takes.
constexpr unsigned COPY_THREADS = 4;
void copy_parallel(void* dst, const void* src, size_t bytes) {
    constexpr size_t MIN_PART = 2u << 20;
    unsigned parts = (unsigned)std::min<size_t>(COPY_THREADS, bytes / MIN_PART);
    if (parts <= 1) {
        std::memcpy(dst, src, bytes);
        return;
    }
    const size_t per = round_up((bytes + parts - 1) / parts, 4096);
    std::vector<std::thread> workers;
    size_t done = 0;
    try {
        for (unsigned k = 1; k < parts; ++k) {
            const size_t off = k * per;
            if (off >= bytes) break;
            const size_t len = std::min(per, bytes - off);
            workers.emplace_back([=] {
                std::memcpy(static_cast<char*>(dst) + off, static_cast<const char*>(src) + off, len);
            });
            done = off + len;
        }
    } catch (...) {  // no thread to be had: the caller's thread copies the rest
        const size_t from = workers.empty() ? per : done;
        if (from < bytes)
            std::memcpy(static_cast<char*>(dst) + from, static_cast<const char*>(src) + from, bytes - from);
    }
    std::memcpy(dst, src, std::min(per, bytes));
    for (std::thread& w : workers) w.join();
}

// Device memory held by the tables of this process, per device, against an optional limit: the
// role of ShardStorageMemory's hard limit (pico-ps/storage/Storage.h:261-289, Storage.cpp:93-98),
// with the device's memory in the place of the host's. Every device allocation of the library goes
// through dev_malloc / dev_free.
constexpr int MAX_DEVICES = 64;
struct DeviceBudget {
    std::mutex mu;
    uint64_t in_use = 0, limit = 0;  // limit 0: none
    std::unordered_map<void*, size_t> sizes;
};
DeviceBudget g_budget[MAX_DEVICES];
thread_local bool g_over_limit = false;  // the calling thread's last dev_malloc failed on the limit

hipError_t dev_malloc(int device, void** p, size_t bytes) {
    g_over_limit = false;
    DeviceBudget& b = g_budget[device];
    {
        std::lock_guard<std::mutex> lk(b.mu);
        if (b.limit && b.in_use + bytes > b.limit) {
            g_over_limit = true;
            return hipErrorOutOfMemory;
        }
        b.in_use += bytes;  // booked first, so that concurrent calls cannot pass the limit together
    }
    hipError_t e = ::hipMalloc(p, bytes);
    std::lock_guard<std::mutex> lk(b.mu);
    if (e != hipSuccess) {
        b.in_use -= bytes;
        return e;
    }
    b.sizes[*p] = bytes;
    return hipSuccess;
}

hipError_t dev_free(int device, void* p) {
    if (!p) return hipSuccess;
    DeviceBudget& b = g_budget[device];
    {
        std::lock_guard<std::mutex> lk(b.mu);
        auto it = b.sizes.find(p);
        if (it != b.sizes.end()) {
            b.in_use -= it->second;
            b.sizes.erase(it);
        }
    }
    return ::hipFree(p);
}

// ---- scratch of the entry point that allocates nothing -------------------------------------------
// pshbm_push_dev_noalloc takes the scratch of a push from this array instead of the table's growing
// workspace. Every device the library runs on holds its own copy until the process ends; in host
// code the array's name is only a stand-in, so the device address is looked up once per device
// (scratch_init) and used from then on.
constexpr size_t NOALLOC_MAX_KEYS = 16384;        // keys per call
constexpr size_t NOALLOC_MAX_FLOATS = 1u << 20;   // keys * dim per call
constexpr size_t NA_WON = 0;                                        // 2 x 17 words, then the sort buffers: one fill clears both
constexpr size_t NA_SORT = 256;
constexpr size_t NA_SORT_ROOM = 1u << 20;
constexpr size_t NA_KEYS5 = NA_SORT + NA_SORT_ROOM;                 // slot, idx, row, srow, sidx
constexpr size_t NA_HDR = NA_KEYS5 + 5 * NOALLOC_MAX_KEYS * 4;
constexpr size_t NA_HDR_ROOM = (NOALLOC_MAX_KEYS / 8 + 1) * sizeof(uint4);
constexpr size_t NA_PVAL = (NA_HDR + NA_HDR_ROOM + 255) / 256 * 256;
constexpr size_t NA_PVAL_ROOM = NOALLOC_MAX_FLOATS + (256u << 10);  // bytes: chunks * 2 * dim floats
constexpr size_t NA_WROW = NA_PVAL + NA_PVAL_ROOM;
constexpr size_t NA_WROW_ROOM = 1024;
constexpr size_t NA_WVAL = NA_WROW + NA_WROW_ROOM;
constexpr size_t NA_WVAL_ROOM = 128u << 10;
constexpr size_t NOALLOC_BYTES = NA_WVAL + NA_WVAL_ROOM;            // about 2.8 MB
static __device__ __align__(256) unsigned char scratch[NOALLOC_BYTES];

std::mutex g_scratch_mu;
unsigned char* g_scratch_ptr[MAX_DEVICES] = {};

// Device address of this device's copy of `scratch`; `device` must be current.
hipError_t scratch_init(int device) {
    std::lock_guard<std::mutex> lk(g_scratch_mu);
    if (g_scratch_ptr[device]) return hipSuccess;
    void* p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess) return e;
    g_scratch_ptr[device] = static_cast<unsigned char*>(p);
    return hipSuccess;
}

}  // namespace

struct pshbm_table {
    pshbm_config cfg{};
    TableDev d{};
    int device = 0;
    uint64_t nbuckets = 0;
    uint32_t row_bits = 0;  // row ids and ROW_NONE differ in their low row_bits bits
    size_t slots_bytes = 0, rows_bytes = 0, keys_bytes = 0;

    uint32_t* h_counters = nullptr;  // pinned, CNT_WORDS
    unsigned long long* d_hist = nullptr;
    unsigned long long* h_hist = nullptr;  // pinned, 17

    // per-batch workspace of the mutating paths
    size_t ws_cap = 0;
    unsigned sort_parity = 0;  // which half of the sort head the next sort uses
    DevBuf ws_slot, ws_row, ws_idx, ws_srow, ws_sidx, ws_sort, ws_hdr, ws_pval, ws_wrow, ws_wval, ws_won;
    unsigned won_parity = 0;  // which half of ws_won the next inserting operation counts into
    // scratch of the partitioned push (batches of PART_MIN_KEYS keys and more)
    DevBuf pt_stage, pt_starts, pt_pstart, pt_psum, pt_new_slot, pt_new_count, pt_ngrad, pt_psize, pt_order, pt_resv;
    size_t part_keys = 0;       // batch size those arrays serve
    // pt_order ranks the partitions of the plan {order_P partitions, order_mask buckets} (0: of none yet)
    uint32_t order_P = 0, order_mask = 0;
    // Row handles (what a pull reports for the push that follows) stay good while no row moves or
    // goes: every erase and clear begins a new epoch.
    uint64_t epoch = 1;

    // staging of the host-pointer entry points
    std::mutex st_mu;
    DevBuf st_keys, st_vals, st_raw;
    // small host-pointer calls go through this pinned buffer: one copy each way instead of the
    // runtime's handling of pageable memory, which costs more than the kernel for a few KB
    void* h_small = nullptr;
    // Host-pointer pulls of different threads share the table (SparsePullOperator.h:188-192): each
    // takes one of these lanes -- a stream with its own staging -- so that their copies and
    // kernels overlap instead of queueing behind one staging buffer. Small host-pointer pushes
    // take a lane for its pinned buffer only: their kernels run on the table's stream one after
    // the other, but a thread waits for its own batch while the next thread's is already queued.
    struct PullLane {
        std::mutex mu;
        hipStream_t stream = nullptr;
        hipEvent_t done = nullptr;  // small pushes: their work on the table's stream has finished
        DevBuf keys, out;
        void* h_small = nullptr;
    };
    static constexpr unsigned PULL_LANES = 4;  // the reference's server runs 4 client-facing threads
    PullLane lanes[PULL_LANES];
    std::atomic<unsigned> next_lane{0};

    // for-each / erase scratch: per-row flags, per-tile counts, row lists, reduction partials;
    // device and pinned copies of {erased, rows left, holes} and of the for-each result
    DevBuf ms_dead, ms_tiles, ms_lists, ms_fe;
    uint32_t* d_info = nullptr;
    uint32_t* h_info = nullptr;
    double* h_fe = nullptr;
    uint64_t tombstones = 0;  // slots holding the marker of an erased key

    // sync-push queue
    DevBuf q_keys, q_grads;
    size_t q_n = 0;

    // bulk staging (load / dump)
    void* pin[2] = {nullptr, nullptr};
    void* dbuf[2] = {nullptr, nullptr};
    hipEvent_t ev_copy[2]{}, ev_done[2]{};

    hipStream_t stream = nullptr, side = nullptr;
    hipEvent_t order_ev{};
    hipStream_t writer_stream = nullptr;      // stream of the last mutating call
    bool has_writer = false;
    // streams, other than the writer's, that have waited for the last mutating call and pulled since
    std::vector<hipStream_t> reader_streams;

    std::shared_mutex mu;
    // Upper bound of the rows handed out, kept without device round trips: the kernels that hand
    // out rows leave {operation number, row count} in the page-locked word h_pub; the bound is the
    // last count seen there (or read back) plus the sizes of the inserting batches enqueued since.
    unsigned long long* h_pub = nullptr;
    uint32_t op_seq = 0;    // number of the last inserting operation enqueued
    uint32_t base_seq = 0;  // rows_base is the row count after this operation
    uint64_t rows_base = 0;
    uint64_t pending_sum = 0;
    std::deque<std::pair<uint32_t, uint32_t>> pending;  // {operation number, keys} enqueued after base_seq

    // optional per-kernel timing (pshbm_profile_*)
    bool prof_on = false;
    std::vector<hipEvent_t> prof_ev;  // start/stop pairs
    std::vector<int> prof_phase;      // phase of each pair in use
};

namespace {

struct DeviceGuard {
    int prev = -1;
    explicit DeviceGuard(int dev) {
        if (hipGetDevice(&prev) != hipSuccess) prev = -1;
        if (prev != dev) (void)hipSetDevice(dev);
    }
    ~DeviceGuard() {
        if (prev >= 0) (void)hipSetDevice(prev);
    }
};

// Message of the calling thread's last failed call: calls on one table may fail on several threads
// at once, so the text is kept per thread, as errno is.
thread_local std::string g_error;

int32_t fail(pshbm_table*, int32_t code, const char* fmt, ...) {
    char buf[512];
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(buf, sizeof buf, fmt, ap);
    va_end(ap);
    g_error = buf;
    return code;
}

int32_t hip_fail(pshbm_table* t, hipError_t e, const char* what) {
    int32_t code = (e == hipErrorOutOfMemory) ? PSHBM_OUT_OF_MEMORY : PSHBM_ERROR;
    if (e == hipErrorOutOfMemory && g_over_limit) {
        g_over_limit = false;
        return fail(t, code, "%s: over the device memory limit (pshbm_set_memory_limit)", what);
    }
    return fail(t, code, "%s: %s", what, hipGetErrorString(e));
}

#define HIP_TRY(t, expr)                                              \
    do {                                                              \
        hipError_t e__ = (expr);                                      \
        if (e__ != hipSuccess) return hip_fail((t), e__, #expr);      \
    } while (0)

// Times `expr` (a kernel launch on stream s) as `phase` when profiling is on.
#define HIP_TRY_PROF(t, s, phase, expr)                               \
    do {                                                              \
        prof_begin((t), (s), (phase));                                \
        hipError_t e__ = (expr);                                      \
        prof_end((t), (s));                                           \
        if (e__ != hipSuccess) return hip_fail((t), e__, #expr);      \
    } while (0)

#define ST_TRY(expr)                          \
    do {                                      \
        int32_t s__ = (expr);                 \
        if (s__ != PSHBM_OK) return s__;      \
    } while (0)

void prof_begin(pshbm_table* t, hipStream_t s, int phase) {
    if (!t->prof_on) return;
    const size_t k = t->prof_phase.size();
    while (t->prof_ev.size() < 2 * (k + 1)) {
        hipEvent_t e = nullptr;
        if (hipEventCreate(&e) != hipSuccess) return;
        t->prof_ev.push_back(e);
    }
    t->prof_phase.push_back(phase);
    (void)hipEventRecord(t->prof_ev[2 * k], s);
}

void prof_end(pshbm_table* t, hipStream_t s) {
    if (!t->prof_on || t->prof_phase.empty()) return;
    (void)hipEventRecord(t->prof_ev[2 * (t->prof_phase.size() - 1) + 1], s);
}

int32_t ensure(pshbm_table* t, DevBuf& b, size_t bytes) {
    if (bytes <= b.bytes) return PSHBM_OK;
    if (b.p) {
        HIP_TRY(t, hipDeviceSynchronize());
        HIP_TRY(t, dev_free(t->device, b.p));
        b.p = nullptr;
        b.bytes = 0;
    }
    size_t want = round_up(bytes + bytes / 4, 256);
    HIP_TRY(t, dev_malloc(t->device, &b.p, want));
    b.bytes = want;
    return PSHBM_OK;
}

// scratch of the mutating paths for a batch of n keys
int32_t ensure_workspace(pshbm_table* t, size_t n) {
    if (n <= t->ws_cap) return PSHBM_OK;
    size_t cap = std::max<size_t>(n, 1024);
    ST_TRY(ensure(t, t->ws_slot, cap * 4));
    ST_TRY(ensure(t, t->ws_idx, cap * 4));
    ST_TRY(ensure(t, t->ws_row, cap * 4));
    ST_TRY(ensure(t, t->ws_srow, cap * 4));
    ST_TRY(ensure(t, t->ws_sidx, cap * 4));
    ST_TRY(ensure(t, t->ws_sort, sort_pairs_temp_bytes(cap)));
    HIP_TRY(t, hipMemset(t->ws_sort.p, 0, sort_pairs_head_bytes()));
    t->sort_parity = 0;
    // partial sums of the segmented reduce: size for the scalar layout, which has more chunks
    SegGeom g1 = seg_geometry(t->d.dim, 1, cap);
    SegGeom g4 = seg_geometry(t->d.dim, (t->d.dim % 4 == 0) ? 4 : 1, cap);
    size_t chunks = std::max(g1.n_chunks, g4.n_chunks);
    ST_TRY(ensure(t, t->ws_hdr, chunks * sizeof(uint4)));
    ST_TRY(ensure(t, t->ws_pval, chunks * 2 * (size_t)t->d.dim * 4));
    ST_TRY(ensure(t, t->ws_wrow, (chunks / 64 + 1) * 4));
    ST_TRY(ensure(t, t->ws_wval, (chunks / 64 + 1) * (size_t)t->d.dim * 4));
    // winner counts per 1024-key block, two arrays used by alternate operations, zero between uses
    ST_TRY(ensure(t, t->ws_won, 2 * (assign_blocks(cap) + 1) * 4));
    HIP_TRY(t, hipMemset(t->ws_won.p, 0, t->ws_won.bytes));
    t->won_parity = 0;
    PartPlan probe_plan;
    if (cap >= PART_MIN_KEYS && part_plan(t->d, std::min(cap, PART_MAX_KEYS), 1.0, &probe_plan)) {
        const size_t pk = std::min(cap, PART_MAX_KEYS);
        const PartSizes z = part_sizes(t->d.dim, pk);
        ST_TRY(ensure(t, t->pt_stage, z.stage));
        ST_TRY(ensure(t, t->pt_starts, z.starts));
        ST_TRY(ensure(t, t->pt_pstart, z.pstart));
        ST_TRY(ensure(t, t->pt_psum, z.psum));
        ST_TRY(ensure(t, t->pt_new_slot, z.new_slot));
        ST_TRY(ensure(t, t->pt_new_count, z.new_count));
        ST_TRY(ensure(t, t->pt_ngrad, z.ngrad));
        ST_TRY(ensure(t, t->pt_psize, z.psize));
        // (of fixed size: allocated by the first batch that qualifies, and cleared then only -- later
        // calls leave them to the kernels that may still be using them)
        const void *order_was = t->pt_order.p, *resv_was = t->pt_resv.p;
        ST_TRY(ensure(t, t->pt_order, z.order));
        ST_TRY(ensure(t, t->pt_resv, z.resv));
        if (t->pt_order.p != order_was) {
            HIP_TRY(t, hipMemset(t->pt_order.p, 0, t->pt_order.bytes));  // (an order of no plan)
            t->order_P = 0;
        }
        if (t->pt_resv.p != resv_was) HIP_TRY(t, hipMemset(t->pt_resv.p, 0, t->pt_resv.bytes));
        t->part_keys = pk;
    }
    t->ws_cap = cap;
    return PSHBM_OK;
}

// Orders this call, on stream s, after the table's earlier calls that it must not overlap. A
// reading call (a pull that inserts nothing) waits for the last mutating call only, so pulls on
// different streams run side by side on the device, as the reference's pulls share a shard
// (SparsePullOperator.h:188-192); a mutating call waits for the last mutating call and for every
// reading call since (the exclusive side of the same lock, SparsePushOperator.h:220).
int32_t begin_op(pshbm_table* t, hipStream_t s, bool reads_only = false) {
    if (reads_only) {
        if (t->has_writer && t->writer_stream == s) return PSHBM_OK;  // stream order
        // one wait per reading stream and mutating call: later pulls on s are behind it already
        if (std::find(t->reader_streams.begin(), t->reader_streams.end(), s) != t->reader_streams.end())
            return PSHBM_OK;
        if (t->has_writer) {
            HIP_TRY(t, hipEventRecord(t->order_ev, t->writer_stream));
            HIP_TRY(t, hipStreamWaitEvent(s, t->order_ev, 0));
        }
        t->reader_streams.push_back(s);  // (also before the first mutating call, which must wait for it)
        return PSHBM_OK;
    }
    if (t->has_writer && t->writer_stream != s) {
        HIP_TRY(t, hipEventRecord(t->order_ev, t->writer_stream));
        HIP_TRY(t, hipStreamWaitEvent(s, t->order_ev, 0));
    }
    for (hipStream_t r : t->reader_streams) {
        if (r == s) continue;
        HIP_TRY(t, hipEventRecord(t->order_ev, r));
        HIP_TRY(t, hipStreamWaitEvent(s, t->order_ev, 0));
    }
    t->reader_streams.clear();
    t->writer_stream = s;
    t->has_writer = true;
    return PSHBM_OK;
}

int32_t read_counters(pshbm_table* t, hipStream_t s) {
    HIP_TRY(t, hipMemcpyAsync(t->h_counters, t->d.counters, CNT_WORDS * 4, hipMemcpyDeviceToHost, s));
    HIP_TRY(t, hipStreamSynchronize(s));
    if (t->h_counters[CNT_SORT_ERR])
        return fail(t, PSHBM_FATAL, "a radix-sort tile timed out waiting for its predecessor: the push it "
                                    "belonged to, and every push since, was not applied (keys they inserted "
                                    "keep their initial values); pshbm_clear resets the table");
    if (t->h_counters[CNT_PART_ERR])
        return fail(t, PSHBM_FATAL, "a push held more entries of one key than a pass of its apply kernel takes (only a "
                                    "pass capacity lowered by pshbm_debug_part_pass_capacity allows that): that push "
                                    "was applied in part; pshbm_clear resets the table");
    return PSHBM_OK;
}

// The table holds exactly `rows` rows and nothing that inserts is in flight.
void set_exact_rows(pshbm_table* t, uint64_t rows) {
    t->rows_base = rows;
    t->base_seq = t->op_seq;
    t->pending.clear();
    t->pending_sum = 0;
}

// Upper bound of the rows handed out, from what the device has published so far.
uint64_t rows_upper_bound(pshbm_table* t) {
    const unsigned long long pub = *static_cast<volatile unsigned long long*>(t->h_pub);
    const uint32_t pseq = (uint32_t)(pub >> 32);
    if ((int32_t)(pseq - t->base_seq) > 0 && (int32_t)(t->op_seq - pseq) >= 0) {
        while (!t->pending.empty() && (int32_t)(t->pending.front().first - pseq) <= 0) {
            t->pending_sum -= t->pending.front().second;
            t->pending.pop_front();
        }
        t->rows_base = (uint32_t)pub;
        t->base_seq = pseq;
    }
    return t->rows_base + t->pending_sum;
}

// Books an inserting batch of n keys: the launches that follow carry its number.
void book_insert(pshbm_table* t, size_t n) {
    ++t->op_seq;
    t->d.op_seq = t->op_seq;
    t->pending.emplace_back(t->op_seq, (uint32_t)n);
    t->pending_sum += n;
}

// Entries per key of the last partitioned push whose apply kernel has run (a tile leaves one entry per
// distinct key it holds: 1 for batches without repeats, about 0.6 for the Zipf batches of the
// benchmark), as that kernel left it in the pinned word; 1 before the first. A hint for the size of
// the next push's partitions, nothing more.
double part_entries_per_key(pshbm_table* t) {
    const unsigned long long st = static_cast<volatile unsigned long long*>(t->h_pub)[1];
    const uint32_t keys = (uint32_t)(st >> 32), entries = (uint32_t)st;
    if (keys == 0 || entries == 0 || entries > keys) return 1.0;
    return (double)entries / (double)keys;
}

// Capacity accounting without a device round trip in the common case: the bound above is exact up
// to the batches still in flight. Only when it would pass the capacity is the exact count read back
// (one stream synchronisation); if even that leaves fewer than n free rows the batch runs in
// checked mode (`*checked`), where the caller inspects the overflow flag after the claim and rolls
// the batch back when it is set.
int32_t reserve_rows(pshbm_table* t, size_t n, hipStream_t s, bool* checked, uint32_t* rows_before) {
    *checked = false;
    if (rows_upper_bound(t) + n <= t->d.max_rows) {
        book_insert(t, n);
        return PSHBM_OK;
    }
    // The bound counts every key of the batches still in flight as a new row. A caller that
    // enqueues faster than the device runs gets many batches ahead, and the bound then passes the
    // capacity long before the table does: wait for the device to publish the row counts of the
    // oldest of them (a poll of the pinned word; the device keeps running, nothing is drained)
    // rather than synchronise the stream. Bounded, because batches recorded into a graph that
    // is being captured publish nothing until the graph runs.
    if (!t->pending.empty()) {
        const auto give_up = std::chrono::steady_clock::now() + std::chrono::milliseconds(20);
        unsigned spins = 0;
        while (!t->pending.empty()) {
            if (rows_upper_bound(t) + n <= t->d.max_rows) {
                book_insert(t, n);
                return PSHBM_OK;
            }
            if ((++spins & 63u) == 0) {
                if (std::chrono::steady_clock::now() > give_up) break;
                std::this_thread::yield();
            }
        }
        if (rows_upper_bound(t) + n <= t->d.max_rows) {
            book_insert(t, n);
            return PSHBM_OK;
        }
    }
    ST_TRY(read_counters(t, s));
    set_exact_rows(t, t->h_counters[CNT_ROWS]);
    book_insert(t, n);
    if (t->rows_base + n <= t->d.max_rows) return PSHBM_OK;
    *checked = true;
    *rows_before = t->h_counters[CNT_ROWS];
    return PSHBM_OK;
}

// After a claim in checked mode: OUT_OF_MEMORY (and the claim undone) if it did not fit.
int32_t settle_rows(pshbm_table* t, const uint32_t* slot_idx, size_t n, hipStream_t s,
                    uint32_t rows_before) {
    ST_TRY(read_counters(t, s));
    if (t->h_counters[CNT_OVERFLOW] || t->h_counters[CNT_ROWS] > t->d.max_rows) {
        HIP_TRY(t, launch_rollback(t->d, slot_idx, n, rows_before, s));
        HIP_TRY(t, hipStreamSynchronize(s));
        set_exact_rows(t, rows_before);
        return fail(t, PSHBM_OUT_OF_MEMORY,
                    "table full: %u keys stored, capacity %u, batch of %zu does not fit",
                    rows_before, t->d.max_rows, n);
    }
    set_exact_rows(t, t->h_counters[CNT_ROWS]);
    return PSHBM_OK;
}

bool has_reserved_key(const uint64_t* keys, size_t n) {
    uint64_t bad = 0;
    for (size_t i = 0; i < n; ++i) bad |= (uint64_t)(keys[i] >= KEY_DELETED);
    return bad != 0;
}

// The probe of a mutating operation: slots of the keys, claiming one for each missing key when
// `insert`, followed by the launch that gives the claimed slots their rows. won_cur / won_next are
// the two arrays of per-block winner counts: the operation counts into one and zeroes the other.
int32_t locate_and_assign(pshbm_table* t, const uint64_t* d_keys, size_t n, uint32_t* slot, uint32_t* idx,
                          uint32_t* row, bool insert, bool init_rows, bool count_dups, uint32_t* won_cur,
                          uint32_t* won_next, size_t won_words, hipStream_t s) {
    if (!insert) {
        HIP_TRY_PROF(t, s, PSHBM_PHASE_LOCATE,
                     launch_locate(t->d, d_keys, n, slot, idx, row, nullptr, count_dups, s));
        return PSHBM_OK;
    }
    HIP_TRY_PROF(t, s, PSHBM_PHASE_LOCATE, launch_locate(t->d, d_keys, n, slot, idx, row, won_cur, count_dups, s));
    HIP_TRY_PROF(t, s, PSHBM_PHASE_ASSIGN_ROWS,
                 launch_assign_rows(t->d, d_keys, n, slot, row, won_cur, won_next, won_words, init_rows, s));
    return PSHBM_OK;
}

// The table's own workspace for the operation that is about to be enqueued (ensure_workspace has
// sized it). The caller flips the halves that alternate between operations once it has used them:
// won_parity after a locate_and_assign that inserts, sort_parity after a sort that used the head.
Workspace table_workspace(pshbm_table* t) {
    Workspace w{};
    w.slot = static_cast<uint32_t*>(t->ws_slot.p);
    w.idx = static_cast<uint32_t*>(t->ws_idx.p);
    w.row = static_cast<uint32_t*>(t->ws_row.p);
    w.srow = static_cast<uint32_t*>(t->ws_srow.p);
    w.sidx = static_cast<uint32_t*>(t->ws_sidx.p);
    w.sort = t->ws_sort.p;
    w.sort_bytes = t->ws_sort.bytes;
    w.sort_parity = t->sort_parity;
    w.hdr = static_cast<uint4*>(t->ws_hdr.p);
    w.pval = static_cast<float*>(t->ws_pval.p);
    w.wrow = static_cast<uint32_t*>(t->ws_wrow.p);
    w.wval = static_cast<float*>(t->ws_wval.p);
    const size_t half = t->ws_won.bytes / 8;  // words per array
    w.won_cur = static_cast<uint32_t*>(t->ws_won.p) + (t->won_parity & 1u) * half;
    w.won_next = static_cast<uint32_t*>(t->ws_won.p) + ((t->won_parity & 1u) ^ 1u) * half;
    w.won_words = half;
    w.part_keys = t->part_keys;
    if (t->part_keys) {
        w.part.stage = static_cast<uint4*>(t->pt_stage.p);
        w.part.starts = static_cast<uint32_t*>(t->pt_starts.p);
        w.part.pstart = static_cast<uint32_t*>(t->pt_pstart.p);
        w.part.psum = static_cast<float*>(t->pt_psum.p);
        w.part.new_slot = static_cast<uint32_t*>(t->pt_new_slot.p);
        w.part.new_count = static_cast<uint32_t*>(t->pt_new_count.p);
        w.part.ngrad = static_cast<float*>(t->pt_ngrad.p);
        w.part.psize = static_cast<uint32_t*>(t->pt_psize.p);
        w.part.order = static_cast<uint32_t*>(t->pt_order.p);
        w.part.resv = static_cast<uint32_t*>(t->pt_resv.p);
    }
    return w;
}

// One push on stream s with the scratch of `w`. *used_sort_head: the sort took the half of the sort
// head that w.sort_parity names (and zeroed the other one).
int32_t push_with(pshbm_table* t, const Workspace& w, const uint64_t* d_keys, const float* d_grads, size_t n,
                  uint32_t flags, hipStream_t s, bool* used_sort_head, bool* used_won, bool* used_part,
                  const uint32_t* d_handles = nullptr) {
    *used_sort_head = false;
    *used_won = false;
    *used_part = false;
    const bool insert = !(flags & PSHBM_PUSH_NO_INSERT);
    const bool unique = (flags & PSHBM_PUSH_ASSUME_UNIQUE) != 0;
    bool checked = false;
    uint32_t rows_before = 0;
    if (insert) ST_TRY(reserve_rows(t, n, s, &checked, &rows_before));
    // A small batch is bound by launches: one workgroup does the whole push in one. (Not when the
    // table is nearly full: undoing a batch that does not fit needs the separate steps.)
    if (!unique && !checked && n <= push_small_max()) {
        HIP_TRY_PROF(t, s, PSHBM_PHASE_PUSH_SMALL, launch_push_small(t->d, d_keys, d_grads, n, insert, s));
        return PSHBM_OK;
    }
    // A large batch is cut into tiles and partitions (push_part.hip): no global sort, one probe per
    // distinct key. (Not in checked mode: it updates rows in the launch that claims slots.)
    PartPlan pl;
    if (!unique && !checked && n <= w.part_keys && part_plan(t->d, n, part_entries_per_key(t), &pl)) {
        *used_part = true;
        // (the other paths look every key up anyway: handles only serve here)
        HIP_TRY_PROF(t, s, PSHBM_PHASE_PART_TILE, launch_part_tile(t->d, pl, w.part, d_keys, d_grads, d_handles, s));
        // The hot keys of one batch are mostly those of the last, and a key's partition is a matter of
        // its hash and the plan: with the same plan, the partitions the last push found full are full again.
        const bool use_order = pl.P >= PART_ORDER_MIN && t->order_P == pl.P && t->order_mask == t->d.bucket_mask;
        HIP_TRY_PROF(t, s, PSHBM_PHASE_PART_APPLY,
                     launch_part_apply(t->d, pl, w.part, d_grads, insert, d_handles != nullptr,
                                       (flags & PSHBM_PUSH_VERIFY_HANDLES) != 0, use_order, s));
        if (insert) {
            const bool make_order = pl.P >= PART_ORDER_MIN;
            HIP_TRY_PROF(t, s, PSHBM_PHASE_PART_INSERT, launch_part_insert(t->d, pl, w.part, d_grads, use_order, make_order, s));
            if (make_order) {
                t->order_P = pl.P;
                t->order_mask = t->d.bucket_mask;
            }
        }
        return PSHBM_OK;
    }
    // Everything after the probe works on row ids: they are dense, so the sort needs fewer bits
    // than for slot indices, the update needs no second look at the hash array, and sorted
    // positions walk the row slab in ascending address order.
    *used_won = insert;  // counted into one array of winner counts, zeroed the other
    ST_TRY(locate_and_assign(t, d_keys, n, w.slot, unique ? nullptr : w.idx, w.row, insert, true, false,
                             w.won_cur, w.won_next, w.won_words, s));
    if (checked) ST_TRY(settle_rows(t, w.slot, n, s, rows_before));
    if (unique) {
        HIP_TRY_PROF(t, s, PSHBM_PHASE_UPDATE_UNIQUE, launch_update_unique(t->d, w.row, n, d_grads, s));
        return PSHBM_OK;
    }
    SortPlan plan;
    // a key inserted by this batch more than once: only the claiming occurrence got the row
    const SortLateKeys late{ROW_PENDING, w.slot, t->d.slots};
    HIP_TRY_PROF(t, s, PSHBM_PHASE_SORT_HIST,
                 sort_begin(w.sort, w.sort_bytes, w.sort_parity, w.row, n, t->row_bits, &plan, s,
                            insert ? &late : nullptr));
    *used_sort_head = plan.uses_head;  // each such sort zeroes the other half for the next
    uint32_t *kin = w.row, *vin = w.idx, *kout = w.srow, *vout = w.sidx;
    for (uint32_t p = 0; p < plan.passes; ++p) {
        HIP_TRY_PROF(t, s, PSHBM_PHASE_SORT_PASS,
                     sort_pass(plan, p, kin, vin, kout, vout, t->d.counters + CNT_SORT_ERR, s));
        std::swap(kin, kout);
        std::swap(vin, vout);
    }
    const bool in_b = (plan.passes & 1u) != 0;
    const uint32_t* fs = in_b ? w.srow : w.row;
    const uint32_t* fi = in_b ? w.sidx : w.idx;
    HIP_TRY_PROF(t, s, PSHBM_PHASE_SEGREDUCE, launch_segreduce(t->d, fs, fi, n, d_grads, w.hdr, w.pval, s));
    HIP_TRY_PROF(t, s, PSHBM_PHASE_FIXUP_WINDOWS,
                 launch_fixup_windows(t->d, n, d_grads, w.hdr, w.pval, w.wrow, w.wval, s));
    HIP_TRY_PROF(t, s, PSHBM_PHASE_FIXUP, launch_fixup(t->d, n, d_grads, w.hdr, w.pval, w.wrow, w.wval, s));
    return PSHBM_OK;
}

int32_t push_locked(pshbm_table* t, const uint64_t* d_keys, const float* d_grads, size_t n,
                    uint32_t flags, hipStream_t s, const uint32_t* d_handles = nullptr) {
    if (n == 0) return PSHBM_OK;
    ST_TRY(begin_op(t, s));
    ST_TRY(ensure_workspace(t, n));
    const Workspace w = table_workspace(t);
    bool used_head = false, used_won = false, used_part = false;
    const int32_t st = push_with(t, w, d_keys, d_grads, n, flags, s, &used_head, &used_won, &used_part, d_handles);
    if (used_head) ++t->sort_parity;
    if (used_won) ++t->won_parity;
    return st;
}

int32_t set_locked(pshbm_table* t, const uint64_t* d_keys, const float* d_values, size_t n,
                   bool count_dups, hipStream_t s) {
    if (n == 0) return PSHBM_OK;
    ST_TRY(begin_op(t, s));
    ST_TRY(ensure_workspace(t, n));
    bool checked = false;
    uint32_t rows_before = 0;
    ST_TRY(reserve_rows(t, n, s, &checked, &rows_before));
    const Workspace w = table_workspace(t);
    ++t->won_parity;
    uint32_t* slot = w.slot;
    ST_TRY(locate_and_assign(t, d_keys, n, slot, nullptr, nullptr, true, false, count_dups, w.won_cur,
                             w.won_next, w.won_words, s));
    if (checked) ST_TRY(settle_rows(t, slot, n, s, rows_before));
    HIP_TRY(t, launch_write_values(t->d, slot, n, d_values, s));
    return PSHBM_OK;
}

int32_t ensure_small(pshbm_table* t) {
    if (!t->h_small) HIP_TRY(t, hipHostMalloc(&t->h_small, SMALL_HOST_BYTES + 4096, hipHostMallocDefault));
    return PSHBM_OK;
}

int32_t ensure_bulk(pshbm_table* t) {
    if (t->pin[0]) return PSHBM_OK;
    for (int k = 0; k < 2; ++k) {
        HIP_TRY(t, hipHostMalloc(&t->pin[k], BULK_CHUNK_BYTES, hipHostMallocDefault));
        HIP_TRY(t, dev_malloc(t->device, &t->dbuf[k], BULK_CHUNK_BYTES));
        HIP_TRY(t, hipEventCreateWithFlags(&t->ev_copy[k], hipEventDisableTiming));
        HIP_TRY(t, hipEventCreateWithFlags(&t->ev_done[k], hipEventDisableTiming));
    }
    return PSHBM_OK;
}

void destroy_impl(pshbm_table* t) {
    DeviceGuard g(t->device);
    (void)hipDeviceSynchronize();
    DevBuf* bufs[] = {&t->ws_slot, &t->ws_row, &t->ws_idx,  &t->ws_srow, &t->ws_sidx, &t->ws_sort, &t->ws_hdr,
                      &t->ws_pval, &t->ws_wrow, &t->ws_wval, &t->ws_won, &t->st_keys, &t->st_vals,  &t->st_raw,
                      &t->ms_dead, &t->ms_tiles, &t->ms_lists, &t->ms_fe,
                      &t->pt_stage, &t->pt_starts, &t->pt_pstart, &t->pt_psum, &t->pt_new_slot, &t->pt_new_count,
                      &t->pt_ngrad, &t->pt_psize, &t->pt_order, &t->pt_resv,
                      &t->q_keys,  &t->q_grads};
    for (DevBuf* b : bufs)
        if (b->p) (void)dev_free(t->device, b->p);
    for (int k = 0; k < 2; ++k) {
        if (t->pin[k]) (void)hipHostFree(t->pin[k]);
        if (t->dbuf[k]) (void)dev_free(t->device, t->dbuf[k]);
        if (t->ev_copy[k]) (void)hipEventDestroy(t->ev_copy[k]);
        if (t->ev_done[k]) (void)hipEventDestroy(t->ev_done[k]);
    }
    if (t->d.slots) (void)dev_free(t->device, t->d.slots);
    if (t->d.rows) (void)dev_free(t->device, t->d.rows);
    if (t->d.row_keys) (void)dev_free(t->device, t->d.row_keys);
    if (t->d.counters) (void)dev_free(t->device, t->d.counters);
    if (t->d.dirty) (void)dev_free(t->device, t->d.dirty);
    if (t->d_hist) (void)dev_free(t->device, t->d_hist);
    if (t->h_counters) (void)hipHostFree(t->h_counters);
    if (t->h_hist) (void)hipHostFree(t->h_hist);
    if (t->h_pub) (void)hipHostFree(t->h_pub);
    if (t->d_info) (void)dev_free(t->device, t->d_info);
    if (t->h_info) (void)hipHostFree(t->h_info);
    if (t->h_fe) (void)hipHostFree(t->h_fe);
    if (t->h_small) (void)hipHostFree(t->h_small);
    for (pshbm_table::PullLane& l : t->lanes) {
        if (l.keys.p) (void)dev_free(t->device, l.keys.p);
        if (l.out.p) (void)dev_free(t->device, l.out.p);
        if (l.h_small) (void)hipHostFree(l.h_small);
        if (l.stream) (void)hipStreamDestroy(l.stream);
        if (l.done) (void)hipEventDestroy(l.done);
    }
    if (t->order_ev) (void)hipEventDestroy(t->order_ev);
    for (hipEvent_t e : t->prof_ev) (void)hipEventDestroy(e);
    if (t->stream) (void)hipStreamDestroy(t->stream);
    if (t->side) (void)hipStreamDestroy(t->side);
    delete t;
}

// ---- for-each / erase ----------------------------------------------------------------------
int32_t check_predicate(pshbm_table* t, const pshbm_predicate* w, pshbm_predicate* out) {
    std::memset(out, 0, sizeof *out);
    out->struct_size = sizeof *out;
    if (!w) return PSHBM_OK;
    if (w->struct_size != sizeof(pshbm_predicate)) return fail(t, PSHBM_INVALID_CONFIG, "predicate: struct_size");
    if (w->n_terms > PSHBM_MAX_TERMS) return fail(t, PSHBM_INVALID_CONFIG, "predicate: more than %d terms", PSHBM_MAX_TERMS);
    for (uint32_t i = 0; i < w->n_terms; ++i) {
        const pshbm_term& m = w->term[i];
        if (m.column != PSHBM_COL_KEY && (m.column < 0 || (uint32_t)m.column >= t->d.vf))
            return fail(t, PSHBM_INVALID_CONFIG, "predicate: term %u names column %d of %u", i, m.column, t->d.vf);
        if (m.cmp < PSHBM_CMP_LT || m.cmp > PSHBM_CMP_PART_NE)
            return fail(t, PSHBM_INVALID_CONFIG, "predicate: term %u has no such comparison", i);
        if ((m.cmp == PSHBM_CMP_PART_EQ || m.cmp == PSHBM_CMP_PART_NE) &&
            (m.column != PSHBM_COL_KEY || m.u == 0 || m.u > 0x7FFFFFFFull))
            return fail(t, PSHBM_INVALID_CONFIG, "predicate: term %u: a partition test needs the key and 1 .. 2^31-1 partitions", i);
        if (m.cmp == PSHBM_CMP_MOD_EQ && (m.column != PSHBM_COL_KEY || m.u == 0))
            return fail(t, PSHBM_INVALID_CONFIG, "predicate: term %u: MOD_EQ needs the key and a modulus", i);
    }
    *out = *w;
    return PSHBM_OK;
}

int32_t ensure_maint(pshbm_table* t) {
    if (!t->d_info) HIP_TRY(t, dev_malloc(t->device, reinterpret_cast<void**>(&t->d_info), 4 * sizeof(uint32_t)));
    if (!t->h_info) HIP_TRY(t, hipHostMalloc(reinterpret_cast<void**>(&t->h_info), 4 * sizeof(uint32_t), hipHostMallocDefault));
    if (!t->h_fe)
        HIP_TRY(t, hipHostMalloc(reinterpret_cast<void**>(&t->h_fe), ((size_t)t->d.vf + 1) * sizeof(double), hipHostMallocDefault));
    return PSHBM_OK;
}

// Hash array rebuilt from the stored keys (the table lock is held).
int32_t compact_locked(pshbm_table* t, hipStream_t s) {
    ST_TRY(read_counters(t, s));
    const uint32_t rows = t->h_counters[CNT_ROWS];
    HIP_TRY(t, hipMemsetAsync(t->d.slots, 0xFF, t->slots_bytes, s));
    HIP_TRY(t, launch_reinsert(t->d, rows, s));
    ST_TRY(read_counters(t, s));
    if (t->h_counters[CNT_OVERFLOW]) return fail(t, PSHBM_FATAL, "compact: the hash array overflowed");
    t->tombstones = 0;
    return PSHBM_OK;
}

// Markers of erased keys occupy slots until the hash array is rebuilt, and inserts never reuse
// them: live keys + markers together must leave the array room to end a probe. The array is
// rebuilt when the markers pass an eighth of the slots, or earlier when a full table (max_rows
// keys) plus the markers would pass 95 % of the slots -- with max_load_factor 0.9 that is a
// twentieth of the slots.
uint64_t tombstone_limit(uint64_t slots, uint64_t max_rows) {
    const uint64_t eighth = slots / 8, ceiling = slots - slots / 20;
    const uint64_t room = ceiling > max_rows ? ceiling - max_rows : 0;
    return room < eighth ? room : eighth;
}

// Removes the rows flagged in ms_dead (one byte per row of the `rows` stored). The lock is held.
int32_t erase_flagged(pshbm_table* t, uint32_t rows, hipStream_t s, uint64_t* erased) {
    uint8_t* dead = static_cast<uint8_t*>(t->ms_dead.p);
    ST_TRY(ensure(t, t->ms_tiles, (erase_tiles(rows) + 1) * 4));
    uint32_t* tiles = static_cast<uint32_t*>(t->ms_tiles.p);
    HIP_TRY(t, launch_erase_count(t->d, rows, dead, tiles, t->d_info, s));
    HIP_TRY(t, hipMemcpyAsync(t->h_info, t->d_info, 4 * sizeof(uint32_t), hipMemcpyDeviceToHost, s));
    HIP_TRY(t, hipStreamSynchronize(s));
    const uint32_t gone = t->h_info[0];
    if (erased) *erased = gone;
    set_exact_rows(t, rows - gone);
    if (gone == 0) return PSHBM_OK;
    ++t->epoch;  // rows move into the holes: handles of earlier pulls are void
    ST_TRY(ensure(t, t->ms_lists, 3 * (size_t)gone * 4));
    HIP_TRY(t, launch_erase_apply(t->d, rows, gone, dead, tiles, t->d_info,
                                  static_cast<uint32_t*>(t->ms_lists.p), s));
    HIP_TRY(t, hipStreamSynchronize(s));
    t->tombstones += gone;
    if (t->tombstones > tombstone_limit(t->nbuckets * 4, t->d.max_rows)) ST_TRY(compact_locked(t, s));
    return PSHBM_OK;
}


}  // namespace

extern "C" {

int32_t pshbm_partition(uint64_t key, int32_t n_partitions) {
    return n_partitions > 0 ? jump_partition(key, n_partitions) : -1;
}

uint32_t pshbm_value_floats(uint32_t dim, int32_t optimizer) {
    switch (optimizer) {
        case PSHBM_OPT_SUM:
        case PSHBM_OPT_SGD: return dim;
        case PSHBM_OPT_ADAGRAD: return 2 * dim;
        case PSHBM_OPT_FTRL: return 3 * dim;
        case PSHBM_OPT_USER: return (1 + pshbm_user::STATE_BLOCKS) * dim;
    }
    return 0;
}

const char* pshbm_last_error(const pshbm_table*) { return g_error.c_str(); }

float pshbm_init_weight(float init_range, uint64_t key, uint32_t column) {
    return init_weight(init_range, key, column);
}

int32_t pshbm_create(const pshbm_config* cfg, pshbm_table** out) {
    if (!cfg || !out) return PSHBM_INVALID_CONFIG;
    *out = nullptr;
    auto bad = [&](const char* m) {
        g_error = m;
        return PSHBM_INVALID_CONFIG;
    };
    if (cfg->struct_size != sizeof(pshbm_config)) return bad("struct_size does not match this library");
    if (cfg->dim == 0 || cfg->dim > MAX_DIM) return bad("dim must be in [1, 16384]");
    const uint32_t vf = pshbm_value_floats(cfg->dim, cfg->optimizer);
    if (vf == 0) return bad("unknown optimizer");
    if (cfg->expected_max_items == 0 || cfg->expected_max_items > 0xFFFFFFF0ull)
        return bad("expected_max_items must be in [1, 2^32-16]");
    float lf = cfg->max_load_factor == 0.0f ? 0.5f : cfg->max_load_factor;
    if (!(lf > 0.0f && lf <= 0.9f)) return bad("max_load_factor must be in (0, 0.9]");
    if (cfg->optimizer == PSHBM_OPT_FTRL && !(cfg->alpha > 0.0f)) return bad("FTRL needs alpha > 0");
    if (!(cfg->init_range >= 0.0f && cfg->init_range <= 3.0e38f)) return bad("init_range must be finite and >= 0");

    int ndev = 0;
    hipError_t e = hipGetDeviceCount(&ndev);
    if (e != hipSuccess || ndev == 0) {
        g_error = std::string("no HIP device: ") + hipGetErrorString(e);
        return PSHBM_ERROR;
    }
    if (cfg->device < 0 || cfg->device >= ndev || cfg->device >= MAX_DEVICES) return bad("device ordinal out of range");

    pshbm_table* t = new (std::nothrow) pshbm_table();
    if (!t) return PSHBM_OUT_OF_MEMORY;
    t->cfg = *cfg;
    t->cfg.max_load_factor = lf;
    t->device = cfg->device;
    DeviceGuard g(t->device);
    if (hipError_t se = scratch_init(t->device); se != hipSuccess) {
        g_error = std::string("hipGetSymbolAddress(scratch): ") + hipGetErrorString(se);
        delete t;
        return PSHBM_ERROR;
    }

    if (hipError_t pe = part_init(); pe != hipSuccess) {
        g_error = std::string("hipFuncSetAttribute (LDS of the partitioned push): ") + hipGetErrorString(pe);
        delete t;
        return PSHBM_ERROR;
    }
    const uint64_t max_rows = cfg->expected_max_items;
    uint64_t want_slots = (uint64_t)((double)max_rows / lf) + 1;
    uint64_t nb = 16;
    while (nb * 4 < want_slots) nb <<= 1;
    if (nb * 4 > (1ull << 31)) {
        delete t;
        return bad("table needs more than 2^31 slots");
    }
    t->nbuckets = nb;
    t->row_bits = 1;
    while ((1ull << t->row_bits) <= max_rows) ++t->row_bits;

    TableDev& d = t->d;
    d.bucket_mask = (uint32_t)(nb - 1);
    d.max_rows = (uint32_t)max_rows;
    d.dim = cfg->dim;
    d.vf = vf;
    d.stride_f = (uint32_t)round_up(vf, 4);
    d.opt = OptParams{cfg->optimizer, (int32_t)(vf / cfg->dim) - 1, cfg->lr, cfg->init_acc, cfg->alpha, cfg->beta,
                      cfg->l1, cfg->l2, cfg->init_range};
    t->slots_bytes = nb * 64;
    t->rows_bytes = max_rows * d.stride_f * 4;
    t->keys_bytes = max_rows * 8;

    auto bail = [&](hipError_t err, const char* what) {
        const bool limit = err == hipErrorOutOfMemory && g_over_limit;
        g_error = std::string(what) + ": " +
                  (limit ? "over the device memory limit (pshbm_set_memory_limit)" : hipGetErrorString(err));
        g_over_limit = false;
        int32_t code = err == hipErrorOutOfMemory ? PSHBM_OUT_OF_MEMORY : PSHBM_ERROR;
        destroy_impl(t);
        return code;
    };
#define CREATE_TRY(expr)                              \
    do {                                              \
        hipError_t e__ = (expr);                      \
        if (e__ != hipSuccess) return bail(e__, #expr); \
    } while (0)
    CREATE_TRY(dev_malloc(t->device, reinterpret_cast<void**>(&d.slots), t->slots_bytes));
    CREATE_TRY(dev_malloc(t->device, reinterpret_cast<void**>(&d.rows), t->rows_bytes));
    CREATE_TRY(dev_malloc(t->device, reinterpret_cast<void**>(&d.row_keys), t->keys_bytes));
    CREATE_TRY(dev_malloc(t->device, reinterpret_cast<void**>(&d.counters), CNT_WORDS * 4));
    if (cfg->track_increment) {
        CREATE_TRY(dev_malloc(t->device, reinterpret_cast<void**>(&d.dirty), round_up(max_rows, 4)));
        CREATE_TRY(hipMemset(d.dirty, 0, round_up(max_rows, 4)));
    }
    CREATE_TRY(dev_malloc(t->device, reinterpret_cast<void**>(&t->d_hist), 17 * 8));
    CREATE_TRY(hipHostMalloc(reinterpret_cast<void**>(&t->h_counters), CNT_WORDS * 4, hipHostMallocDefault));
    CREATE_TRY(hipHostMalloc(reinterpret_cast<void**>(&t->h_hist), 17 * 8, hipHostMallocDefault));
    CREATE_TRY(hipHostMalloc(reinterpret_cast<void**>(&t->h_pub), 16, hipHostMallocDefault));
    t->h_pub[0] = 0;
    t->h_pub[1] = 0;
    d.pub = t->h_pub;
    d.part_stat = t->h_pub + 1;
    CREATE_TRY(hipStreamCreateWithFlags(&t->stream, hipStreamNonBlocking));
    CREATE_TRY(hipStreamCreateWithFlags(&t->side, hipStreamNonBlocking));
    for (pshbm_table::PullLane& l : t->lanes) {
        CREATE_TRY(hipStreamCreateWithFlags(&l.stream, hipStreamNonBlocking));
        CREATE_TRY(hipEventCreateWithFlags(&l.done, hipEventDisableTiming));
    }
    CREATE_TRY(hipEventCreateWithFlags(&t->order_ev, hipEventDisableTiming));
    CREATE_TRY(hipMemsetAsync(d.slots, 0xFF, t->slots_bytes, t->stream));
    CREATE_TRY(hipMemsetAsync(d.counters, 0, CNT_WORDS * 4, t->stream));
    CREATE_TRY(hipStreamSynchronize(t->stream));
#undef CREATE_TRY
    int32_t st = ensure_workspace(t, cfg->max_batch ? cfg->max_batch : 65536);
    if (st != PSHBM_OK) {
        destroy_impl(t);
        return st;
    }
    *out = t;
    return PSHBM_OK;
}

int32_t pshbm_destroy(pshbm_table* t) {
    if (!t) return PSHBM_OK;
    destroy_impl(t);
    return PSHBM_OK;
}

// ---- pull ------------------------------------------------------------------------------------
static int32_t pull_dev_impl(pshbm_table* t, const uint64_t* d_keys, size_t n, float* d_out_rows,
                             uint8_t* d_hit, uint32_t* d_handles, uint64_t* epoch, uint32_t flags, void* stream) {
    if (!t) return PSHBM_INVALID_ID;
    if (n == 0) {
        if (epoch) {
            std::shared_lock<std::shared_mutex> rl(t->mu);
            *epoch = t->epoch;
        }
        return PSHBM_OK;
    }
    if (!d_keys || !d_out_rows) return fail(t, PSHBM_ERROR, "pull: null buffer");
    if (n > 0x7FFFFFFFull) return fail(t, PSHBM_ERROR, "pull: batch larger than 2^31-1 keys");
    DeviceGuard g(t->device);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const bool insert = (flags & PSHBM_PULL_INSERT_ON_MISS) && !t->cfg.read_only;
    std::unique_lock<std::shared_mutex> lk(t->mu);
    ST_TRY(begin_op(t, s, !insert));
    if (!insert) {
        if (epoch) *epoch = t->epoch;
        HIP_TRY_PROF(t, s, PSHBM_PHASE_PULL, launch_pull(t->d, d_keys, n, d_out_rows, d_hit, d_handles, s));
        return PSHBM_OK;
    }
    ST_TRY(ensure_workspace(t, n));
    bool checked = false;
    uint32_t rows_before = 0;
    ST_TRY(reserve_rows(t, n, s, &checked, &rows_before));
    const Workspace w = table_workspace(t);
    ++t->won_parity;
    uint32_t* slot = w.slot;
    ST_TRY(locate_and_assign(t, d_keys, n, slot, nullptr, nullptr, true, true, false, w.won_cur, w.won_next,
                             w.won_words, s));
    if (checked) ST_TRY(settle_rows(t, slot, n, s, rows_before));
    if (epoch) *epoch = t->epoch;
    HIP_TRY_PROF(t, s, PSHBM_PHASE_GATHER, launch_gather_slots(t->d, d_keys, slot, n, d_out_rows, d_hit, d_handles, s));
    return PSHBM_OK;
}

int32_t pshbm_pull_dev(pshbm_table* t, const uint64_t* d_keys, size_t n, float* d_out_rows,
                       uint8_t* d_hit, uint32_t flags, void* stream) {
    return pull_dev_impl(t, d_keys, n, d_out_rows, d_hit, nullptr, nullptr, flags, stream);
}

int32_t pshbm_pull_dev_handles(pshbm_table* t, const uint64_t* d_keys, size_t n, float* d_out_rows,
                               uint8_t* d_hit, uint32_t* d_handles, uint64_t* epoch, uint32_t flags,
                               void* stream) {
    if (t && (!d_handles || !epoch)) return fail(t, PSHBM_ERROR, "pull_handles: null handle buffer or epoch");
    return pull_dev_impl(t, d_keys, n, d_out_rows, d_hit, d_handles, epoch, flags, stream);
}

// A lane that is free, else the next one in turn; held until `lock` goes.
static pshbm_table::PullLane* take_lane(pshbm_table* t, std::unique_lock<std::mutex>& lock) {
    const unsigned first = t->next_lane.fetch_add(1, std::memory_order_relaxed) % pshbm_table::PULL_LANES;
    for (unsigned k = 0; k < pshbm_table::PULL_LANES; ++k) {
        pshbm_table::PullLane& c = t->lanes[(first + k) % pshbm_table::PULL_LANES];
        std::unique_lock<std::mutex> trial(c.mu, std::try_to_lock);
        if (trial.owns_lock()) {
            lock = std::move(trial);
            return &c;
        }
    }
    lock = std::unique_lock<std::mutex>(t->lanes[first].mu);
    return &t->lanes[first];
}

static int32_t lane_pinned(pshbm_table* t, pshbm_table::PullLane* lane) {
    if (!lane->h_small)
        HIP_TRY(t, hipHostMalloc(&lane->h_small, SMALL_HOST_BYTES + 4096, hipHostMallocDefault));
    return PSHBM_OK;
}

int32_t pshbm_pull(pshbm_table* t, const uint64_t* keys, size_t n, float* out_rows, uint8_t* hit,
                   uint32_t flags) {
    if (!t) return PSHBM_INVALID_ID;
    if (n == 0) return PSHBM_OK;
    if (!keys || !out_rows) return fail(t, PSHBM_ERROR, "pull: null buffer");
    if (has_reserved_key(keys, n)) return fail(t, PSHBM_ERROR, "pull: reserved key in batch");
    DeviceGuard g(t->device);
    std::unique_lock<std::mutex> ll;
    pshbm_table::PullLane* lane = take_lane(t, ll);
    const size_t key_bytes = n * 8, out_bytes = n * (size_t)t->d.dim * 4;
    hipStream_t s = lane->stream;
    const size_t key_room = round_up(key_bytes, 256);
    if (key_room + out_bytes + n <= SMALL_HOST_BYTES) {
        // Buffers of the caller that are page-locked already (pshbm_host_alloc) are used as they
        // lie: the kernel reads the keys from them and writes the rows into them.
        if (is_pinned_host(keys, key_bytes) && is_pinned_host(out_rows, out_bytes) && (!hit || is_pinned_host(hit, n))) {
            ST_TRY(pshbm_pull_dev(t, keys, n, out_rows, hit, flags, s));
            HIP_TRY(t, hipStreamSynchronize(s));
            return PSHBM_OK;
        }
        ST_TRY(lane_pinned(t, lane));
        // The kernel reads the keys from the pinned buffer and writes rows and hit mask into it:
        // page-locked host memory is mapped into the device's address space, and for a few
        // hundred KB the link's latency inside one kernel is cheaper than two copy commands.
        char* h = static_cast<char*>(lane->h_small);
        std::memcpy(h, keys, key_bytes);
        ST_TRY(pshbm_pull_dev(t, reinterpret_cast<const uint64_t*>(h), n, reinterpret_cast<float*>(h + key_room),
                              reinterpret_cast<uint8_t*>(h + key_room + out_bytes), flags, s));
        HIP_TRY(t, hipStreamSynchronize(s));
        std::memcpy(out_rows, h + key_room, out_bytes);
        if (hit) std::memcpy(hit, h + key_room + out_bytes, n);
        return PSHBM_OK;
    }
    ST_TRY(ensure(t, lane->keys, key_bytes));
    ST_TRY(ensure(t, lane->out, out_bytes + n));  // the hit mask follows the rows
    const uint64_t* d_keys = static_cast<const uint64_t*>(lane->keys.p);
    float* d_rows = static_cast<float*>(lane->out.p);
    uint8_t* d_hit = static_cast<uint8_t*>(lane->out.p) + out_bytes;
    HIP_TRY(t, hipMemcpyAsync(lane->keys.p, keys, key_bytes, hipMemcpyHostToDevice, s));
    ST_TRY(pshbm_pull_dev(t, d_keys, n, d_rows, d_hit, flags, s));
    HIP_TRY(t, hipMemcpyAsync(out_rows, d_rows, out_bytes, hipMemcpyDeviceToHost, s));
    if (hit) HIP_TRY(t, hipMemcpyAsync(hit, d_hit, n, hipMemcpyDeviceToHost, s));
    HIP_TRY(t, hipStreamSynchronize(s));
    return PSHBM_OK;
}

// ---- push ------------------------------------------------------------------------------------
int32_t pshbm_push_dev(pshbm_table* t, const uint64_t* d_keys, const float* d_grads, size_t n,
                       uint32_t flags, void* stream) {
    if (!t) return PSHBM_INVALID_ID;
    if (n == 0) return PSHBM_OK;
    if (!d_keys || !d_grads) return fail(t, PSHBM_ERROR, "push: null buffer");
    if (n > MAX_PUSH_BATCH) return fail(t, PSHBM_ERROR, "push: batch larger than 2^30-1 keys");
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    return push_locked(t, d_keys, d_grads, n, flags, static_cast<hipStream_t>(stream));
}

int32_t pshbm_push_dev_handles(pshbm_table* t, const uint64_t* d_keys, const float* d_grads,
                               const uint32_t* d_handles, uint64_t epoch, size_t n, uint32_t flags,
                               void* stream) {
    if (!t) return PSHBM_INVALID_ID;
    if (n == 0) return PSHBM_OK;
    if (!d_keys || !d_grads) return fail(t, PSHBM_ERROR, "push: null buffer");
    if (n > MAX_PUSH_BATCH) return fail(t, PSHBM_ERROR, "push: batch larger than 2^30-1 keys");
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    // handles of another epoch say nothing any more: the push looks every key up, as pshbm_push_dev does
    const uint32_t* h = (d_handles && epoch == t->epoch) ? d_handles : nullptr;
    return push_locked(t, d_keys, d_grads, n, flags, static_cast<hipStream_t>(stream), h);
}

// The same push with its scratch in the library's fixed device array: nothing is allocated, by this
// call or by anything it calls. One array per device, shared by every table on it.
int32_t pshbm_push_dev_noalloc(pshbm_table* t, const uint64_t* d_keys, const float* d_grads, size_t n,
                               uint32_t flags, void* stream) {
    if (!t) return PSHBM_INVALID_ID;
    if (n == 0) return PSHBM_OK;
    if (!d_keys || !d_grads) return fail(t, PSHBM_ERROR, "push_noalloc: null buffer");
    if (n > NOALLOC_MAX_KEYS || n * (size_t)t->d.dim > NOALLOC_MAX_FLOATS)
        return fail(t, PSHBM_ERROR, "push_noalloc: at most %zu keys and %zu gradient floats per call (got %zu keys of dim %u)",
                    NOALLOC_MAX_KEYS, NOALLOC_MAX_FLOATS, n, t->d.dim);
    DeviceGuard g(t->device);
    hipStream_t s = static_cast<hipStream_t>(stream);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    std::lock_guard<std::mutex> sk(g_scratch_mu);  // one enqueue at a time per process; overlap on the device is the caller's to avoid
    unsigned char* base = g_scratch_ptr[t->device];
    if (!base) return fail(t, PSHBM_FATAL, "push_noalloc: the scratch array was not set up for device %d", t->device);
    // what this batch needs of the array, by the same geometry the kernels use
    const SegGeom g1 = seg_geometry(t->d.dim, 1, n);
    const SegGeom g4 = seg_geometry(t->d.dim, (t->d.dim % 4 == 0) ? 4 : 1, n);
    const size_t chunks = std::max(g1.n_chunks, g4.n_chunks);
    if (sort_pairs_temp_bytes(n) > NA_SORT_ROOM || chunks * sizeof(uint4) > NA_HDR_ROOM ||
        chunks * 2 * (size_t)t->d.dim * 4 > NA_PVAL_ROOM || (chunks / 64 + 1) * 4 > NA_WROW_ROOM ||
        (chunks / 64 + 1) * (size_t)t->d.dim * 4 > NA_WVAL_ROOM || 2 * (assign_blocks(n) + 1) * 4 > NA_SORT - NA_WON)
        return fail(t, PSHBM_ERROR, "push_noalloc: a batch of %zu keys of dim %u does not fit the fixed scratch", n, t->d.dim);
    ST_TRY(begin_op(t, s));
    Workspace w{};
    uint32_t* k5 = reinterpret_cast<uint32_t*>(base + NA_KEYS5);
    w.slot = k5;
    w.idx = k5 + NOALLOC_MAX_KEYS;
    w.row = k5 + 2 * NOALLOC_MAX_KEYS;
    w.srow = k5 + 3 * NOALLOC_MAX_KEYS;
    w.sidx = k5 + 4 * NOALLOC_MAX_KEYS;
    w.sort = base + NA_SORT;
    w.sort_bytes = NA_SORT_ROOM;
    w.sort_parity = 0;
    w.hdr = reinterpret_cast<uint4*>(base + NA_HDR);
    w.pval = reinterpret_cast<float*>(base + NA_PVAL);
    w.wrow = reinterpret_cast<uint32_t*>(base + NA_WROW);
    w.wval = reinterpret_cast<float*>(base + NA_WVAL);
    w.won_words = assign_blocks(NOALLOC_MAX_KEYS) + 1;
    w.won_cur = reinterpret_cast<uint32_t*>(base + NA_WON);
    w.won_next = w.won_cur + w.won_words;
    // The array keeps what the last call left: the winner counts and the sort's digit totals must
    // start at zero (a fill kernel, not a memset: the call may be recorded into a graph).
    HIP_TRY(t, launch_fill_u32(reinterpret_cast<uint32_t*>(base + NA_WON), (NA_SORT + sort_pairs_head_bytes()) / 4, 0u, s));
    const bool prof = t->prof_on;  // the per-kernel timers create events on demand
    t->prof_on = false;
    bool used_head = false, used_won = false, used_part = false;  // (w.part_keys = 0: never the partitioned path)
    const int32_t st = push_with(t, w, d_keys, d_grads, n, flags, s, &used_head, &used_won, &used_part);
    t->prof_on = prof;
    return st;
}

// Keys and their n x `floats` values from host memory to where kernels on stream s can read them:
// *dk / *dv. Larger batches are copied into st_keys / st_vals. Small ones are copied into the pinned
// buffer (unless the caller's buffers are page-locked themselves) and read from there by the
// kernels (page-locked memory is mapped into the device's address space; the buffer is in use
// until the stream has been waited for). The caller holds st_mu.
static int32_t stage_keys_values(pshbm_table* t, const uint64_t* keys, const float* vals, size_t n,
                                 size_t floats, hipStream_t s, const uint64_t** dk, const float** dv) {
    const size_t key_bytes = n * 8, val_bytes = n * floats * 4;
    const size_t key_room = round_up(key_bytes, 256);
    if (key_room + val_bytes <= SMALL_HOST_BYTES) {
        if (is_pinned_host(keys, key_bytes) && is_pinned_host(vals, val_bytes)) {  // usable as they lie
            *dk = keys;
            *dv = vals;
            return PSHBM_OK;
        }
        ST_TRY(ensure_small(t));
        char* h = static_cast<char*>(t->h_small);
        std::memcpy(h, keys, key_bytes);
        std::memcpy(h + key_room, vals, val_bytes);
        *dk = reinterpret_cast<const uint64_t*>(h);
        *dv = reinterpret_cast<const float*>(h + key_room);
        return PSHBM_OK;
    }
    ST_TRY(ensure(t, t->st_keys, key_bytes));
    ST_TRY(ensure(t, t->st_vals, val_bytes));
    HIP_TRY(t, hipMemcpyAsync(t->st_keys.p, keys, key_bytes, hipMemcpyHostToDevice, s));
    HIP_TRY(t, hipMemcpyAsync(t->st_vals.p, vals, val_bytes, hipMemcpyHostToDevice, s));
    *dk = static_cast<const uint64_t*>(t->st_keys.p);
    *dv = static_cast<const float*>(t->st_vals.p);
    return PSHBM_OK;
}

int32_t pshbm_push(pshbm_table* t, const uint64_t* keys, const float* grads, size_t n, uint32_t flags) {
    if (!t) return PSHBM_INVALID_ID;
    if (n == 0) return PSHBM_OK;
    if (!keys || !grads) return fail(t, PSHBM_ERROR, "push: null buffer");
    if (has_reserved_key(keys, n)) return fail(t, PSHBM_ERROR, "push: reserved key in batch");
    DeviceGuard g(t->device);
    hipStream_t s = t->stream;
    const size_t key_bytes = n * 8, val_bytes = n * (size_t)t->d.dim * 4;
    const size_t key_room = round_up(key_bytes, 256);
    if (key_room + val_bytes <= SMALL_HOST_BYTES) {
        // the kernels read the batch from a lane's pinned buffer (or from the caller's buffers, if
        // those are page-locked already); the thread waits for its own batch only, so the next
        // thread's push is queued behind it meanwhile
        std::unique_lock<std::mutex> ll;
        pshbm_table::PullLane* lane = take_lane(t, ll);
        const uint64_t* dk = keys;
        const float* dv = grads;
        if (!(is_pinned_host(keys, key_bytes) && is_pinned_host(grads, val_bytes))) {
            ST_TRY(lane_pinned(t, lane));
            char* h = static_cast<char*>(lane->h_small);
            std::memcpy(h, keys, key_bytes);
            std::memcpy(h + key_room, grads, val_bytes);
            dk = reinterpret_cast<const uint64_t*>(h);
            dv = reinterpret_cast<const float*>(h + key_room);
        }
        int32_t st = pshbm_push_dev(t, dk, dv, n, flags, s);
        HIP_TRY(t, hipEventRecord(lane->done, s));
        HIP_TRY(t, hipEventSynchronize(lane->done));
        return st;
    }
    std::lock_guard<std::mutex> sl(t->st_mu);
    const uint64_t* dk = nullptr;
    const float* dv = nullptr;
    ST_TRY(stage_keys_values(t, keys, grads, n, t->d.dim, s, &dk, &dv));
    int32_t st = pshbm_push_dev(t, dk, dv, n, flags, s);
    HIP_TRY(t, hipStreamSynchronize(s));
    return st;
}

// Copies n wire pairs {uint64 key, dim floats} to the device and splits them there into the staged
// key and gradient arrays (st_keys, st_vals): the path of large blocks. The caller holds st_mu.
static int32_t stage_pairs(pshbm_table* t, const void* pairs, size_t n, size_t stride, const char* what) {
    if (!pairs) return fail(t, PSHBM_ERROR, "%s: null buffer", what);
    const size_t used = 8 + (size_t)t->d.dim * 4;
    if (stride < used || stride % 4) return fail(t, PSHBM_ERROR, "%s: bad stride %zu", what, stride);
    const char* p = static_cast<const char*>(pairs);
    for (size_t i = 0; i < n; ++i) {
        uint64_t k;
        std::memcpy(&k, p + i * stride, 8);
        if (k >= KEY_DELETED) return fail(t, PSHBM_ERROR, "%s: reserved key in batch", what);
    }
    ST_TRY(ensure(t, t->st_keys, n * 8));
    ST_TRY(ensure(t, t->st_vals, n * (size_t)t->d.dim * 4));
    hipStream_t s = t->stream;
    ST_TRY(ensure(t, t->st_raw, n * stride));
    HIP_TRY(t, hipMemcpyAsync(t->st_raw.p, pairs, n * stride, hipMemcpyHostToDevice, s));
    HIP_TRY(t, launch_unpack_records(static_cast<const uint32_t*>(t->st_raw.p), n,
                                     (uint32_t)(stride / 4), t->d.dim,
                                     static_cast<uint64_t*>(t->st_keys.p),
                                     static_cast<float*>(t->st_vals.p), s));
    return PSHBM_OK;
}

// n wire pairs {uint64 key, dim floats} split into a key array and a gradient array on the host.
static int32_t split_pairs(pshbm_table* t, const void* pairs, size_t n, size_t stride, char* keys_out,
                           char* grads_out, const char* what) {
    const char* p = static_cast<const char*>(pairs);
    const size_t row_bytes = (size_t)t->d.dim * 4;
    for (size_t i = 0; i < n; ++i) {
        uint64_t k;
        std::memcpy(&k, p + i * stride, 8);
        if (k >= KEY_DELETED) return fail(t, PSHBM_ERROR, "%s: reserved key in batch", what);
        std::memcpy(keys_out + i * 8, &k, 8);
        std::memcpy(grads_out + i * row_bytes, p + i * stride + 8, row_bytes);
    }
    return PSHBM_OK;
}

int32_t pshbm_push_pairs(pshbm_table* t, const void* pairs, size_t n, size_t stride, uint32_t flags) {
    if (!t) return PSHBM_INVALID_ID;
    if (n == 0) return PSHBM_OK;
    DeviceGuard g(t->device);
    const size_t key_room = round_up(n * 8, 256), val_bytes = n * (size_t)t->d.dim * 4;
    if (pairs && stride >= 8 + (size_t)t->d.dim * 4 && stride % 4 == 0 && key_room + val_bytes <= SMALL_HOST_BYTES) {
        // a small block is split into keys and gradients on its way into a lane's pinned buffer
        std::unique_lock<std::mutex> ll;
        pshbm_table::PullLane* lane = take_lane(t, ll);
        ST_TRY(lane_pinned(t, lane));
        char* h = static_cast<char*>(lane->h_small);
        int32_t st = split_pairs(t, pairs, n, stride, h, h + key_room, "push_pairs");
        if (st != PSHBM_OK) return st;
        st = pshbm_push_dev(t, reinterpret_cast<const uint64_t*>(h),
                                    reinterpret_cast<const float*>(h + key_room), n, flags, t->stream);
        HIP_TRY(t, hipEventRecord(lane->done, t->stream));
        HIP_TRY(t, hipEventSynchronize(lane->done));
        return st;
    }
    std::lock_guard<std::mutex> sl(t->st_mu);
    ST_TRY(stage_pairs(t, pairs, n, stride, "push_pairs"));
    int32_t st = pshbm_push_dev(t, static_cast<const uint64_t*>(t->st_keys.p),
                                static_cast<const float*>(t->st_vals.p), n, flags, t->stream);
    HIP_TRY(t, hipStreamSynchronize(t->stream));
    return st;
}

int32_t pshbm_queue_pairs(pshbm_table* t, const void* pairs, size_t n, size_t stride) {
    if (!t) return PSHBM_INVALID_ID;
    if (n == 0) return PSHBM_OK;
    DeviceGuard g(t->device);
    const size_t key_room = round_up(n * 8, 256), val_bytes = n * (size_t)t->d.dim * 4;
    if (pairs && stride >= 8 + (size_t)t->d.dim * 4 && stride % 4 == 0 && key_room + val_bytes <= SMALL_HOST_BYTES) {
        std::unique_lock<std::mutex> ll;
        pshbm_table::PullLane* lane = take_lane(t, ll);
        ST_TRY(lane_pinned(t, lane));
        char* h = static_cast<char*>(lane->h_small);
        int32_t st = split_pairs(t, pairs, n, stride, h, h + key_room, "queue_pairs");
        if (st != PSHBM_OK) return st;
        st = pshbm_queue_dev(t, reinterpret_cast<const uint64_t*>(h), reinterpret_cast<const float*>(h + key_room), n,
                             t->stream);
        HIP_TRY(t, hipEventRecord(lane->done, t->stream));
        HIP_TRY(t, hipEventSynchronize(lane->done));
        return st;
    }
    std::lock_guard<std::mutex> sl(t->st_mu);
    ST_TRY(stage_pairs(t, pairs, n, stride, "queue_pairs"));
    int32_t st = pshbm_queue_dev(t, static_cast<const uint64_t*>(t->st_keys.p),
                                 static_cast<const float*>(t->st_vals.p), n, t->stream);
    HIP_TRY(t, hipStreamSynchronize(t->stream));
    return st;
}

// ---- sync push: queue + store ----------------------------------------------------------------
int32_t pshbm_queue_dev(pshbm_table* t, const uint64_t* d_keys, const float* d_grads, size_t n,
                        void* stream) {
    if (!t) return PSHBM_INVALID_ID;
    if (n == 0) return PSHBM_OK;
    if (!d_keys || !d_grads) return fail(t, PSHBM_ERROR, "queue: null buffer");
    DeviceGuard g(t->device);
    hipStream_t s = static_cast<hipStream_t>(stream);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    if (t->q_n + n > MAX_PUSH_BATCH) return fail(t, PSHBM_ERROR, "queue: more than 2^30-1 keys queued");
    ST_TRY(begin_op(t, s));
    const size_t gb = (size_t)t->d.dim * 4;
    const size_t need = t->q_n + n;
    if (need * 8 > t->q_keys.bytes) {  // grow, keeping what is queued
        DevBuf nk, ng;
        size_t cap = std::max(need * 2, (size_t)65536);
        HIP_TRY(t, hipStreamSynchronize(s));
        HIP_TRY(t, dev_malloc(t->device, &nk.p, cap * 8));
        nk.bytes = cap * 8;
        hipError_t e = dev_malloc(t->device, &ng.p, cap * gb);
        if (e != hipSuccess) {
            (void)dev_free(t->device, nk.p);
            return hip_fail(t, e, "queue: hipMalloc");
        }
        ng.bytes = cap * gb;
        if (t->q_n) {
            HIP_TRY(t, hipMemcpy(nk.p, t->q_keys.p, t->q_n * 8, hipMemcpyDeviceToDevice));
            HIP_TRY(t, hipMemcpy(ng.p, t->q_grads.p, t->q_n * gb, hipMemcpyDeviceToDevice));
        }
        if (t->q_keys.p) (void)dev_free(t->device, t->q_keys.p);
        if (t->q_grads.p) (void)dev_free(t->device, t->q_grads.p);
        t->q_keys = nk;
        t->q_grads = ng;
    }
    // (the host-pointer entry points hand their pinned or pageable buffers straight to these copies)
    HIP_TRY(t, hipMemcpyAsync(static_cast<uint64_t*>(t->q_keys.p) + t->q_n, d_keys, n * 8,
                              hipMemcpyDefault, s));
    HIP_TRY(t, hipMemcpyAsync(static_cast<char*>(t->q_grads.p) + t->q_n * gb, d_grads, n * gb,
                              hipMemcpyDefault, s));
    t->q_n += n;
    return PSHBM_OK;
}

int32_t pshbm_queue(pshbm_table* t, const uint64_t* keys, const float* grads, size_t n) {
    if (!t) return PSHBM_INVALID_ID;
    if (n == 0) return PSHBM_OK;
    if (!keys || !grads) return fail(t, PSHBM_ERROR, "queue: null buffer");
    if (has_reserved_key(keys, n)) return fail(t, PSHBM_ERROR, "queue: reserved key in batch");
    DeviceGuard g(t->device);
    hipStream_t s = t->stream;
    const size_t key_bytes = n * 8, val_bytes = n * (size_t)t->d.dim * 4;
    const size_t key_room = round_up(key_bytes, 256);
    if (key_room + val_bytes <= SMALL_HOST_BYTES) {  // through a lane's pinned buffer, as a small push
        std::unique_lock<std::mutex> ll;
        pshbm_table::PullLane* lane = take_lane(t, ll);
        ST_TRY(lane_pinned(t, lane));
        char* h = static_cast<char*>(lane->h_small);
        std::memcpy(h, keys, key_bytes);
        std::memcpy(h + key_room, grads, val_bytes);
        int32_t st = pshbm_queue_dev(t, reinterpret_cast<const uint64_t*>(h),
                                     reinterpret_cast<const float*>(h + key_room), n, s);
        HIP_TRY(t, hipEventRecord(lane->done, s));
        HIP_TRY(t, hipEventSynchronize(lane->done));
        return st;
    }
    std::lock_guard<std::mutex> sl(t->st_mu);
    int32_t st = pshbm_queue_dev(t, keys, grads, n, s);  // copied from the caller's memory into the queue
    HIP_TRY(t, hipStreamSynchronize(s));
    return st;
}

int32_t pshbm_queued(pshbm_table* t, uint64_t* n) {
    if (!t || !n) return PSHBM_INVALID_ID;
    std::shared_lock<std::shared_mutex> lk(t->mu);
    *n = t->q_n;
    return PSHBM_OK;
}

int32_t pshbm_store_dev(pshbm_table* t, uint32_t flags, void* stream) {
    if (!t) return PSHBM_INVALID_ID;
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    const size_t n = t->q_n;
    t->q_n = 0;
    return push_locked(t, static_cast<const uint64_t*>(t->q_keys.p),
                       static_cast<const float*>(t->q_grads.p), n,
                       flags & ~PSHBM_PUSH_ASSUME_UNIQUE, static_cast<hipStream_t>(stream));
}

int32_t pshbm_store(pshbm_table* t, uint32_t flags) {
    if (!t) return PSHBM_INVALID_ID;
    DeviceGuard g(t->device);
    int32_t st = pshbm_store_dev(t, flags, t->stream);
    HIP_TRY(t, hipStreamSynchronize(t->stream));
    return st;
}

// ---- set / load / dump / iterate ---------------------------------------------------------------
int32_t pshbm_set_dev(pshbm_table* t, const uint64_t* d_keys, const float* d_values, size_t n,
                      void* stream) {
    if (!t) return PSHBM_INVALID_ID;
    if (n == 0) return PSHBM_OK;
    if (!d_keys || !d_values) return fail(t, PSHBM_ERROR, "set: null buffer");
    if (n > 0x7FFFFFFFull) return fail(t, PSHBM_ERROR, "set: batch larger than 2^31-1 keys");
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    return set_locked(t, d_keys, d_values, n, false, static_cast<hipStream_t>(stream));
}

int32_t pshbm_set(pshbm_table* t, const uint64_t* keys, const float* values, size_t n) {
    if (!t) return PSHBM_INVALID_ID;
    if (n == 0) return PSHBM_OK;
    if (!keys || !values) return fail(t, PSHBM_ERROR, "set: null buffer");
    if (has_reserved_key(keys, n)) return fail(t, PSHBM_ERROR, "set: reserved key in batch");
    DeviceGuard g(t->device);
    std::lock_guard<std::mutex> sl(t->st_mu);
    hipStream_t s = t->stream;
    const uint64_t* dk = nullptr;
    const float* dv = nullptr;
    ST_TRY(stage_keys_values(t, keys, values, n, t->d.vf, s, &dk, &dv));
    int32_t st = pshbm_set_dev(t, dk, dv, n, s);
    HIP_TRY(t, hipStreamSynchronize(s));
    return st;
}

int32_t pshbm_load(pshbm_table* t, const void* records, size_t n, uint32_t flags) {
    if (!t) return PSHBM_INVALID_ID;
    if (n == 0) return PSHBM_OK;
    if (!records) return fail(t, PSHBM_ERROR, "load: null buffer");
    DeviceGuard g(t->device);
    std::lock_guard<std::mutex> sl(t->st_mu);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    ST_TRY(ensure_bulk(t));
    const size_t rec = 8 + (size_t)t->d.vf * 4;
    const size_t per_chunk = BULK_CHUNK_BYTES / rec;
    if (per_chunk == 0) return fail(t, PSHBM_ERROR, "load: record larger than the staging chunk");
    ST_TRY(ensure(t, t->st_keys, per_chunk * 8));
    ST_TRY(ensure(t, t->st_vals, per_chunk * (size_t)t->d.vf * 4));
    ST_TRY(ensure_workspace(t, per_chunk));
    hipStream_t s = t->stream;
    ST_TRY(begin_op(t, s));
    const bool unique = (flags & PSHBM_LOAD_UNIQUE) != 0;
    // the probe counts the records it skips for their reserved key, and the keys it finds stored
    HIP_TRY(t, hipMemsetAsync(t->d.counters + CNT_BADKEY, 0, 4, s));
    if (unique) HIP_TRY(t, hipMemsetAsync(t->d.counters + CNT_DUP, 0, 4, s));
    // page-locked records go to the device as they lie; others through the pinned staging pair
    const bool direct = is_pinned_host(records, n * rec);
    const char* src = static_cast<const char*>(records);
    int32_t status = PSHBM_OK;
    size_t chunk = 0;
    for (size_t off = 0; off < n; off += per_chunk, ++chunk) {
        const size_t cnt = std::min(per_chunk, n - off);
        const int k = (int)(chunk & 1);
        const char* rp = src + off * rec;
        // the host stays two chunks ahead of the device; then pin[k] has left the host, too
        if (chunk >= 2) HIP_TRY(t, hipEventSynchronize(t->ev_copy[k]));
        if (!direct) copy_parallel(t->pin[k], rp, cnt * rec);
        if (chunk >= 2) HIP_TRY(t, hipStreamWaitEvent(t->side, t->ev_done[k], 0));  // device chunk consumed
        HIP_TRY(t, hipMemcpyAsync(t->dbuf[k], direct ? static_cast<const void*>(rp) : t->pin[k], cnt * rec,
                                  hipMemcpyHostToDevice, t->side));
        HIP_TRY(t, hipEventRecord(t->ev_copy[k], t->side));
        HIP_TRY(t, hipStreamWaitEvent(s, t->ev_copy[k], 0));
        HIP_TRY(t, launch_unpack_records(static_cast<const uint32_t*>(t->dbuf[k]), cnt,
                                         (uint32_t)(rec / 4), t->d.vf,
                                         static_cast<uint64_t*>(t->st_keys.p),
                                         static_cast<float*>(t->st_vals.p), s));
        HIP_TRY(t, hipEventRecord(t->ev_done[k], s));
        status = set_locked(t, static_cast<const uint64_t*>(t->st_keys.p),
                            static_cast<const float*>(t->st_vals.p), cnt, unique, s);
        if (status != PSHBM_OK) break;
    }
    HIP_TRY(t, hipStreamSynchronize(t->side));
    ST_TRY(read_counters(t, s));
    if (status != PSHBM_OK) return status;
    if (t->h_counters[CNT_BADKEY])
        return fail(t, PSHBM_ERROR, "load: %u records with a reserved key were skipped",
                    t->h_counters[CNT_BADKEY]);
    if (unique && t->h_counters[CNT_DUP])
        return fail(t, PSHBM_ERROR, "load: %u keys were already present or repeated",
                    t->h_counters[CNT_DUP]);
    return PSHBM_OK;
}

// Records of rows [first, first + count) of the slab, or, with row_list (device), of the rows
// row_list[first .. first + count), whose marks are cleared on the way.
static int32_t dump_range(pshbm_table* t, size_t first, size_t count, void* records,
                          const uint32_t* row_list = nullptr) {
    ST_TRY(ensure_bulk(t));
    const size_t rec = 8 + (size_t)t->d.vf * 4;
    const size_t per_chunk = BULK_CHUNK_BYTES / rec;
    if (per_chunk == 0) return fail(t, PSHBM_ERROR, "dump: record larger than the staging chunk");
    hipStream_t s = t->stream;
    char* dst = static_cast<char*>(records);
    // a page-locked destination is written by the copy engine itself; any other one gets its
    // records from the pinned staging pair, two chunks behind the kernels
    const bool direct = is_pinned_host(records, count * rec);
    size_t chunk = 0;
    size_t pending_off[2] = {0, 0}, pending_cnt[2] = {0, 0};
    for (size_t off = 0; off < count; off += per_chunk, ++chunk) {
        const size_t cnt = std::min(per_chunk, count - off);
        const int k = (int)(chunk & 1);
        if (chunk >= 2) {  // the chunk that used this pair of buffers
            // (the host waits also when it has nothing to copy: it stays two chunks ahead of the
            // device instead of queueing the whole dump at once)
            HIP_TRY(t, hipEventSynchronize(t->ev_copy[k]));
            if (!direct) copy_parallel(dst + pending_off[k] * rec, t->pin[k], pending_cnt[k] * rec);
        }
        if (row_list)
            HIP_TRY(t, launch_pack_rows(t->d, row_list + first + off, cnt, static_cast<uint32_t*>(t->dbuf[k]), s));
        else
            HIP_TRY(t, launch_pack_records(t->d, (uint32_t)(first + off), cnt,
                                           static_cast<uint32_t*>(t->dbuf[k]), s));
        HIP_TRY(t, hipEventRecord(t->ev_done[k], s));
        HIP_TRY(t, hipStreamWaitEvent(t->side, t->ev_done[k], 0));
        HIP_TRY(t, hipMemcpyAsync(direct ? static_cast<void*>(dst + off * rec) : t->pin[k], t->dbuf[k], cnt * rec,
                                  hipMemcpyDeviceToHost, t->side));
        HIP_TRY(t, hipEventRecord(t->ev_copy[k], t->side));
        // dbuf[k] (and pin[k]) are reused two chunks later, after ev_copy[k]
        pending_off[k] = off;
        pending_cnt[k] = cnt;
    }
    const size_t nchunks = chunk;
    if (!direct) {
        for (size_t c = (nchunks >= 2 ? nchunks - 2 : 0); c < nchunks; ++c) {
            const int k = (int)(c & 1);
            HIP_TRY(t, hipEventSynchronize(t->ev_copy[k]));
            copy_parallel(dst + pending_off[k] * rec, t->pin[k], pending_cnt[k] * rec);
        }
    }
    HIP_TRY(t, hipStreamSynchronize(t->side));
    HIP_TRY(t, hipStreamSynchronize(s));
    return PSHBM_OK;
}

int32_t pshbm_iterate(pshbm_table* t, size_t offset, size_t batch, void* records, size_t* n_out) {
    if (!t || !n_out) return PSHBM_INVALID_ID;
    *n_out = 0;
    DeviceGuard g(t->device);
    std::lock_guard<std::mutex> sl(t->st_mu);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    ST_TRY(begin_op(t, t->stream));
    ST_TRY(read_counters(t, t->stream));
    const size_t size = t->h_counters[CNT_ROWS];
    if (offset >= size || batch == 0) return PSHBM_OK;
    if (!records) return fail(t, PSHBM_ERROR, "iterate: null buffer");
    const size_t cnt = std::min(batch, size - offset);
    ST_TRY(dump_range(t, offset, cnt, records));
    *n_out = cnt;
    return PSHBM_OK;
}

int32_t pshbm_iterate_keys(pshbm_table* t, size_t offset, size_t batch, uint64_t* keys, size_t* n_out) {
    if (!t || !n_out) return PSHBM_INVALID_ID;
    *n_out = 0;
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    hipStream_t s = t->stream;
    ST_TRY(begin_op(t, s));
    ST_TRY(read_counters(t, s));
    const size_t size = t->h_counters[CNT_ROWS];
    if (offset >= size || batch == 0) return PSHBM_OK;
    if (!keys) return fail(t, PSHBM_ERROR, "iterate_keys: null buffer");
    const size_t cnt = std::min(batch, size - offset);
    // the keys of the rows lie in one array, in the order of the records
    HIP_TRY(t, hipMemcpyAsync(keys, t->d.row_keys + offset, cnt * 8, hipMemcpyDeviceToHost, s));
    HIP_TRY(t, hipStreamSynchronize(s));
    *n_out = cnt;
    return PSHBM_OK;
}

int32_t pshbm_dump(pshbm_table* t, void* records, size_t capacity_records, size_t* n_out) {
    if (!t || !n_out) return PSHBM_INVALID_ID;
    *n_out = 0;
    DeviceGuard g(t->device);
    std::lock_guard<std::mutex> sl(t->st_mu);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    ST_TRY(begin_op(t, t->stream));
    ST_TRY(read_counters(t, t->stream));
    const size_t size = t->h_counters[CNT_ROWS];
    if (size == 0) return PSHBM_OK;
    if (capacity_records < size)
        return fail(t, PSHBM_ERROR, "dump: buffer holds %zu records, table has %zu", capacity_records, size);
    if (!records) return fail(t, PSHBM_ERROR, "dump: null buffer");
    ST_TRY(dump_range(t, 0, size, records));
    *n_out = size;
    return PSHBM_OK;
}

// ---- clear / size / stats ----------------------------------------------------------------------
// ---- for-each / erase ------------------------------------------------------------------------
int32_t pshbm_for_each(pshbm_table* t, const pshbm_predicate* where, uint64_t* count, double* column_sums) {
    if (!t) return PSHBM_INVALID_ID;
    if (!count) return fail(t, PSHBM_ERROR, "for_each: null count");
    pshbm_predicate pred;
    ST_TRY(check_predicate(t, where, &pred));
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    hipStream_t s = t->stream;
    ST_TRY(begin_op(t, s));
    ST_TRY(ensure_maint(t));
    ST_TRY(read_counters(t, s));
    const uint32_t rows = t->h_counters[CNT_ROWS];
    const uint32_t vf = t->d.vf;
    *count = 0;
    if (column_sums) std::fill(column_sums, column_sums + vf, 0.0);
    if (rows == 0) return PSHBM_OK;
    ST_TRY(ensure(t, t->ms_fe, for_each_scratch_bytes(t->d)));
    double* scratch = static_cast<double*>(t->ms_fe.p);
    HIP_TRY(t, launch_for_each(t->d, rows, pred, scratch, s));
    HIP_TRY(t, hipMemcpyAsync(t->h_fe, scratch, ((size_t)vf + 1) * sizeof(double), hipMemcpyDeviceToHost, s));
    HIP_TRY(t, hipStreamSynchronize(s));
    *count = (uint64_t)t->h_fe[vf];
    if (column_sums) std::copy(t->h_fe, t->h_fe + vf, column_sums);
    return PSHBM_OK;
}

int32_t pshbm_for_each_write(pshbm_table* t, const pshbm_predicate* where, const pshbm_update* what,
                             uint64_t* count) {
    if (!t) return PSHBM_INVALID_ID;
    if (count) *count = 0;
    if (t->cfg.read_only) return fail(t, PSHBM_ERROR, "for_each_write: the table is read-only");
    if (!what || what->struct_size != sizeof(pshbm_update))
        return fail(t, PSHBM_INVALID_CONFIG, "for_each_write: update struct_size");
    if (what->op != PSHBM_UPD_AFFINE && what->op != PSHBM_UPD_CLAMP)
        return fail(t, PSHBM_INVALID_CONFIG, "for_each_write: no such operation");
    if ((uint64_t)what->first_column + what->n_columns > t->d.vf)
        return fail(t, PSHBM_INVALID_CONFIG, "for_each_write: columns %u..%u of %u", what->first_column,
                    what->first_column + what->n_columns, t->d.vf);
    pshbm_predicate pred;
    ST_TRY(check_predicate(t, where, &pred));
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    hipStream_t s = t->stream;
    ST_TRY(begin_op(t, s));
    ST_TRY(ensure_maint(t));
    ST_TRY(read_counters(t, s));
    const uint32_t rows = t->h_counters[CNT_ROWS];
    if (rows == 0) return PSHBM_OK;
    ST_TRY(ensure(t, t->ms_fe, for_each_scratch_bytes(t->d)));
    double* scratch = static_cast<double*>(t->ms_fe.p);
    HIP_TRY(t, launch_for_each_write(t->d, rows, pred, *what, scratch, s));
    HIP_TRY(t, hipMemcpyAsync(t->h_fe, scratch, sizeof(double), hipMemcpyDeviceToHost, s));
    HIP_TRY(t, hipStreamSynchronize(s));
    if (count) *count = (uint64_t)t->h_fe[0];
    return PSHBM_OK;
}

int32_t pshbm_erase_if(pshbm_table* t, const pshbm_predicate* where, uint64_t* erased) {
    if (!t) return PSHBM_INVALID_ID;
    if (t->cfg.read_only) return fail(t, PSHBM_ERROR, "erase_if: the table is read-only");
    pshbm_predicate pred;
    ST_TRY(check_predicate(t, where, &pred));
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    hipStream_t s = t->stream;
    ST_TRY(begin_op(t, s));
    ST_TRY(ensure_maint(t));
    ST_TRY(read_counters(t, s));
    const uint32_t rows = t->h_counters[CNT_ROWS];
    if (erased) *erased = 0;
    if (rows == 0) return PSHBM_OK;
    ST_TRY(ensure(t, t->ms_dead, round_up(rows, 4)));
    HIP_TRY(t, launch_mark_pred(t->d, rows, pred, static_cast<uint8_t*>(t->ms_dead.p), s));
    return erase_flagged(t, rows, s, erased);
}

int32_t pshbm_erase_dev(pshbm_table* t, const uint64_t* d_keys, size_t n, uint64_t* erased, void* stream) {
    if (!t) return PSHBM_INVALID_ID;
    if (erased) *erased = 0;
    if (n == 0) return PSHBM_OK;
    if (!d_keys) return fail(t, PSHBM_ERROR, "erase: null buffer");
    if (n > 0x7FFFFFFFull) return fail(t, PSHBM_ERROR, "erase: batch larger than 2^31-1 keys");
    if (t->cfg.read_only) return fail(t, PSHBM_ERROR, "erase: the table is read-only");
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    hipStream_t s = static_cast<hipStream_t>(stream);
    ST_TRY(begin_op(t, s));
    ST_TRY(ensure_maint(t));
    ST_TRY(ensure_workspace(t, n));
    ST_TRY(read_counters(t, s));
    const uint32_t rows = t->h_counters[CNT_ROWS];
    if (rows == 0) return PSHBM_OK;
    ST_TRY(ensure(t, t->ms_dead, round_up(rows, 4)));
    uint8_t* dead = static_cast<uint8_t*>(t->ms_dead.p);
    HIP_TRY(t, hipMemsetAsync(dead, 0, round_up(rows, 4), s));
    uint32_t* slot = static_cast<uint32_t*>(t->ws_slot.p);
    uint32_t* row = static_cast<uint32_t*>(t->ws_row.p);
    HIP_TRY(t, launch_locate(t->d, d_keys, n, slot, nullptr, row, nullptr, false, s));
    HIP_TRY(t, launch_mark_rows(row, n, rows, dead, s));
    return erase_flagged(t, rows, s, erased);
}

int32_t pshbm_erase(pshbm_table* t, const uint64_t* keys, size_t n, uint64_t* erased) {
    if (!t) return PSHBM_INVALID_ID;
    if (erased) *erased = 0;
    if (n == 0) return PSHBM_OK;
    if (!keys) return fail(t, PSHBM_ERROR, "erase: null buffer");
    if (has_reserved_key(keys, n)) return fail(t, PSHBM_ERROR, "erase: reserved key in batch");
    DeviceGuard g(t->device);
    std::lock_guard<std::mutex> sl(t->st_mu);
    ST_TRY(ensure(t, t->st_keys, n * 8));
    hipStream_t s = t->stream;
    HIP_TRY(t, hipMemcpyAsync(t->st_keys.p, keys, n * 8, hipMemcpyHostToDevice, s));
    return pshbm_erase_dev(t, static_cast<const uint64_t*>(t->st_keys.p), n, erased, s);
}

int32_t pshbm_compact(pshbm_table* t) {
    if (!t) return PSHBM_INVALID_ID;
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    hipStream_t s = t->stream;
    ST_TRY(begin_op(t, s));
    return compact_locked(t, s);
}

// ---- increment -------------------------------------------------------------------------------
// Marked rows counted (and, with `list`, listed in ms_lists). The lock is held.
static int32_t increment_scan(pshbm_table* t, hipStream_t s, bool list, uint32_t* marked) {
    *marked = 0;
    ST_TRY(ensure_maint(t));
    ST_TRY(read_counters(t, s));
    const uint32_t rows = t->h_counters[CNT_ROWS];
    if (rows == 0) return PSHBM_OK;
    ST_TRY(ensure(t, t->ms_tiles, (erase_tiles(rows) + 1) * 4));
    uint32_t* tiles = static_cast<uint32_t*>(t->ms_tiles.p);
    HIP_TRY(t, launch_erase_count(t->d, rows, t->d.dirty, tiles, t->d_info, s, false));
    HIP_TRY(t, hipMemcpyAsync(t->h_info, t->d_info, 4 * sizeof(uint32_t), hipMemcpyDeviceToHost, s));
    HIP_TRY(t, hipStreamSynchronize(s));
    *marked = t->h_info[0];
    if (list && *marked) {
        ST_TRY(ensure(t, t->ms_lists, (size_t)*marked * 4));
        HIP_TRY(t, launch_flag_list(rows, t->d.dirty, tiles, static_cast<uint32_t*>(t->ms_lists.p), s));
    }
    return PSHBM_OK;
}

int32_t pshbm_increment_size(pshbm_table* t, uint64_t* n) {
    if (!t || !n) return PSHBM_INVALID_ID;
    *n = 0;
    if (!t->d.dirty) return fail(t, PSHBM_ERROR, "the table was created without track_increment");
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    ST_TRY(begin_op(t, t->stream));
    uint32_t marked = 0;
    ST_TRY(increment_scan(t, t->stream, false, &marked));
    *n = marked;
    return PSHBM_OK;
}

int32_t pshbm_take_increment(pshbm_table* t, void* records, size_t capacity_records, size_t* n_out) {
    if (!t || !n_out) return PSHBM_INVALID_ID;
    *n_out = 0;
    if (!t->d.dirty) return fail(t, PSHBM_ERROR, "the table was created without track_increment");
    DeviceGuard g(t->device);
    std::lock_guard<std::mutex> sl(t->st_mu);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    ST_TRY(begin_op(t, t->stream));
    uint32_t marked = 0;
    ST_TRY(increment_scan(t, t->stream, true, &marked));
    *n_out = marked;
    if (marked == 0) return PSHBM_OK;
    if (marked > capacity_records || !records)
        return fail(t, PSHBM_ERROR, "take_increment: %u records, room for %zu", marked, capacity_records);
    return dump_range(t, 0, marked, records, static_cast<const uint32_t*>(t->ms_lists.p));
}

int32_t pshbm_set_hyperparameters(pshbm_table* t, const pshbm_hyperparameters* hp) {
    if (!t) return PSHBM_INVALID_ID;
    if (!hp || hp->struct_size != sizeof(pshbm_hyperparameters))
        return fail(t, PSHBM_INVALID_CONFIG, "set_hyperparameters: struct_size");
    if (t->cfg.optimizer == PSHBM_OPT_FTRL && !(hp->alpha > 0.0f))
        return fail(t, PSHBM_INVALID_CONFIG, "set_hyperparameters: FTRL needs alpha > 0");
    // kernels take the parameters by value at launch: calls already queued keep the old ones
    std::unique_lock<std::shared_mutex> lk(t->mu);
    t->cfg.lr = hp->lr;
    t->cfg.init_acc = hp->init_acc;
    t->cfg.alpha = hp->alpha;
    t->cfg.beta = hp->beta;
    t->cfg.l1 = hp->l1;
    t->cfg.l2 = hp->l2;
    t->d.opt = OptParams{t->cfg.optimizer, t->d.opt.states, hp->lr, hp->init_acc, hp->alpha, hp->beta, hp->l1, hp->l2,
                         t->cfg.init_range};
    return PSHBM_OK;
}

int32_t pshbm_reserve(pshbm_table* t, uint64_t expected_max_items) {
    if (!t) return PSHBM_INVALID_ID;
    if (expected_max_items > 0xFFFFFFF0ull)
        return fail(t, PSHBM_INVALID_CONFIG, "reserve: at most 2^32-16 keys");
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    if (expected_max_items <= t->d.max_rows) return PSHBM_OK;
    hipStream_t s = t->stream;
    ST_TRY(begin_op(t, s));
    ST_TRY(read_counters(t, s));  // waits for everything queued on the table so far
    const uint32_t rows = t->h_counters[CNT_ROWS];
    const uint64_t max_rows = expected_max_items;
    uint64_t want_slots = (uint64_t)((double)max_rows / t->cfg.max_load_factor) + 1;
    uint64_t nb = 16;
    while (nb * 4 < want_slots) nb <<= 1;
    if (nb * 4 > (1ull << 31)) return fail(t, PSHBM_INVALID_CONFIG, "reserve: the table would need more than 2^31 slots");
    const size_t stride = t->d.stride_f;
    const size_t slots_bytes = nb * 64, rows_bytes = max_rows * stride * 4, keys_bytes = max_rows * 8;
    const size_t dirty_bytes = round_up(max_rows, 4);
    uint4* n_slots = nullptr;
    float* n_rows = nullptr;
    uint64_t* n_keys = nullptr;
    uint8_t* n_dirty = nullptr;
    auto undo = [&](hipError_t e, const char* what) {
        if (n_slots) (void)dev_free(t->device, n_slots);
        if (n_rows) (void)dev_free(t->device, n_rows);
        if (n_keys) (void)dev_free(t->device, n_keys);
        if (n_dirty) (void)dev_free(t->device, n_dirty);
        return hip_fail(t, e, what);
    };
    hipError_t e;
    if ((e = dev_malloc(t->device, reinterpret_cast<void**>(&n_slots), slots_bytes)) != hipSuccess) return undo(e, "reserve: hash array");
    if ((e = dev_malloc(t->device, reinterpret_cast<void**>(&n_rows), rows_bytes)) != hipSuccess) return undo(e, "reserve: rows");
    if ((e = dev_malloc(t->device, reinterpret_cast<void**>(&n_keys), keys_bytes)) != hipSuccess) return undo(e, "reserve: row keys");
    if (t->d.dirty && (e = dev_malloc(t->device, reinterpret_cast<void**>(&n_dirty), dirty_bytes)) != hipSuccess)
        return undo(e, "reserve: marks");
    // rows keep their numbers: the slab is copied as it is and the hash array rebuilt from row_keys
    if ((e = hipMemsetAsync(n_slots, 0xFF, slots_bytes, s)) != hipSuccess) return undo(e, "reserve: fill");
    if (rows) {
        if ((e = hipMemcpyAsync(n_rows, t->d.rows, (size_t)rows * stride * 4, hipMemcpyDeviceToDevice, s)) != hipSuccess)
            return undo(e, "reserve: copy rows");
        if ((e = hipMemcpyAsync(n_keys, t->d.row_keys, (size_t)rows * 8, hipMemcpyDeviceToDevice, s)) != hipSuccess)
            return undo(e, "reserve: copy keys");
    }
    if (n_dirty) {
        if ((e = hipMemsetAsync(n_dirty, 0, dirty_bytes, s)) != hipSuccess) return undo(e, "reserve: marks");
        if (rows && (e = hipMemcpyAsync(n_dirty, t->d.dirty, rows, hipMemcpyDeviceToDevice, s)) != hipSuccess)
            return undo(e, "reserve: copy marks");
    }
    if ((e = hipStreamSynchronize(s)) != hipSuccess) return undo(e, "reserve: copy");
    uint4* o_slots = t->d.slots;
    float* o_rows = t->d.rows;
    uint64_t* o_keys = t->d.row_keys;
    uint8_t* o_dirty = t->d.dirty;
    t->d.slots = n_slots;
    t->d.rows = n_rows;
    t->d.row_keys = n_keys;
    t->d.dirty = n_dirty;
    t->d.bucket_mask = (uint32_t)(nb - 1);
    t->d.max_rows = (uint32_t)max_rows;
    t->nbuckets = nb;
    t->slots_bytes = slots_bytes;
    t->rows_bytes = rows_bytes;
    t->keys_bytes = keys_bytes;
    t->cfg.expected_max_items = max_rows;
    t->row_bits = 1;
    while ((1ull << t->row_bits) <= max_rows) ++t->row_bits;
    t->tombstones = 0;
    (void)dev_free(t->device, o_slots);
    (void)dev_free(t->device, o_rows);
    (void)dev_free(t->device, o_keys);
    if (o_dirty) (void)dev_free(t->device, o_dirty);
    HIP_TRY(t, launch_reinsert(t->d, rows, s));
    ST_TRY(read_counters(t, s));
    if (t->h_counters[CNT_OVERFLOW]) return fail(t, PSHBM_FATAL, "reserve: the hash array overflowed");
    return PSHBM_OK;
}

int32_t pshbm_clear(pshbm_table* t) {
    if (!t) return PSHBM_INVALID_ID;
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    hipStream_t s = t->stream;
    ST_TRY(begin_op(t, s));
    HIP_TRY(t, hipMemsetAsync(t->d.slots, 0xFF, t->slots_bytes, s));
    HIP_TRY(t, hipMemsetAsync(t->d.counters, 0, CNT_WORDS * 4, s));
    if (t->d.dirty) HIP_TRY(t, hipMemsetAsync(t->d.dirty, 0, round_up(t->d.max_rows, 4), s));
    HIP_TRY(t, hipStreamSynchronize(s));
    set_exact_rows(t, 0);
    t->tombstones = 0;
    ++t->epoch;
    return PSHBM_OK;
}

int32_t pshbm_size(pshbm_table* t, uint64_t* n) {
    if (!t || !n) return PSHBM_INVALID_ID;
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    ST_TRY(begin_op(t, t->stream));
    ST_TRY(read_counters(t, t->stream));
    set_exact_rows(t, t->h_counters[CNT_ROWS]);
    *n = t->h_counters[CNT_ROWS];
    return PSHBM_OK;
}

int32_t pshbm_set_memory_limit(int32_t device, uint64_t bytes) {
    if (device < 0 || device >= MAX_DEVICES) return PSHBM_INVALID_ID;
    std::lock_guard<std::mutex> lk(g_budget[device].mu);
    g_budget[device].limit = bytes;
    return PSHBM_OK;
}

int32_t pshbm_device_memory(int32_t device, uint64_t* in_use, uint64_t* limit) {
    if (device < 0 || device >= MAX_DEVICES) return PSHBM_INVALID_ID;
    std::lock_guard<std::mutex> lk(g_budget[device].mu);
    if (in_use) *in_use = g_budget[device].in_use;
    if (limit) *limit = g_budget[device].limit;
    return PSHBM_OK;
}

int32_t pshbm_memory_usage(pshbm_table* t, uint64_t* bytes) {
    if (!t || !bytes) return PSHBM_INVALID_ID;
    std::shared_lock<std::shared_mutex> lk(t->mu);
    *bytes = t->slots_bytes + t->rows_bytes + t->keys_bytes;
    return PSHBM_OK;
}

int32_t pshbm_get_stats(pshbm_table* t, pshbm_stats* out) {
    if (!t || !out) return PSHBM_INVALID_ID;
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    hipStream_t s = t->stream;
    ST_TRY(begin_op(t, s));
    ST_TRY(read_counters(t, s));
    const uint32_t rows = t->h_counters[CNT_ROWS];
    HIP_TRY(t, hipMemsetAsync(t->d_hist, 0, 17 * 8, s));
    HIP_TRY(t, launch_probe_hist(t->d, rows, t->d_hist, s));
    HIP_TRY(t, hipMemcpyAsync(t->h_hist, t->d_hist, 17 * 8, hipMemcpyDeviceToHost, s));
    HIP_TRY(t, hipStreamSynchronize(s));
    std::memset(out, 0, sizeof *out);
    out->size = rows;
    out->capacity = t->d.max_rows;
    out->slots = t->nbuckets * 4;
    out->memory_usage = t->slots_bytes + t->rows_bytes + t->keys_bytes;
    out->load_factor = (double)rows / (double)(t->nbuckets * 4);
    for (int i = 0; i < 16; ++i) out->probe_hist[i] = t->h_hist[i];
    out->max_probe = t->h_hist[16];
    return PSHBM_OK;
}

int32_t pshbm_profile_enable(pshbm_table* t, int32_t on) {
    if (!t) return PSHBM_INVALID_ID;
    std::unique_lock<std::shared_mutex> lk(t->mu);
    t->prof_on = on != 0;
    return PSHBM_OK;
}

int32_t pshbm_profile_read(pshbm_table* t, pshbm_profile* out) {
    if (!t || !out) return PSHBM_INVALID_ID;
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    std::memset(out, 0, sizeof *out);
    for (size_t k = 0; k < t->prof_phase.size(); ++k) {
        HIP_TRY(t, hipEventSynchronize(t->prof_ev[2 * k + 1]));
        float ms = 0.f;
        HIP_TRY(t, hipEventElapsedTime(&ms, t->prof_ev[2 * k], t->prof_ev[2 * k + 1]));
        const int ph = t->prof_phase[k];
        out->ms[ph] += ms;
        out->launches[ph] += 1;
    }
    t->prof_phase.clear();
    return PSHBM_OK;
}

int32_t pshbm_debug_sort_spin_limit(uint32_t polls) {
    sort_set_spin_limit(polls);
    return PSHBM_OK;
}

int32_t pshbm_debug_sort_pairs(int32_t device, uint32_t* d_keys, uint32_t* d_vals, uint32_t* d_keys_tmp,
                               uint32_t* d_vals_tmp, size_t n, uint32_t key_bits, int32_t* result_in_tmp,
                               void* stream) {
    if (!d_keys || !d_vals || !d_keys_tmp || !d_vals_tmp || !result_in_tmp || key_bits == 0 || key_bits > 32)
        return PSHBM_ERROR;
    if (n == 0) {
        *result_in_tmp = 0;
        return PSHBM_OK;
    }
    DeviceGuard g(device);
    hipStream_t s = static_cast<hipStream_t>(stream);
    const size_t temp_bytes = sort_pairs_temp_bytes(n);
    void* temp = nullptr;
    uint32_t* err = nullptr;
    if (hipMalloc(&temp, temp_bytes) != hipSuccess) return PSHBM_OUT_OF_MEMORY;
    if (hipMalloc(reinterpret_cast<void**>(&err), 4) != hipSuccess) {
        (void)hipFree(temp);
        return PSHBM_OUT_OF_MEMORY;
    }
    bool in_b = false;
    uint32_t h_err = 0;
    hipError_t e = hipMemsetAsync(temp, 0, sort_pairs_head_bytes(), s);
    if (e == hipSuccess) e = hipMemsetAsync(err, 0, 4, s);
    if (e == hipSuccess) e = sort_pairs(temp, temp_bytes, 0, d_keys, d_keys_tmp, d_vals, d_vals_tmp, n, key_bits, &in_b, err, s);
    if (e == hipSuccess) e = hipMemcpyAsync(&h_err, err, 4, hipMemcpyDeviceToHost, s);
    if (e == hipSuccess) e = hipStreamSynchronize(s);
    (void)hipFree(temp);
    (void)hipFree(err);
    *result_in_tmp = in_b ? 1 : 0;
    if (e != hipSuccess) return PSHBM_ERROR;
    return h_err ? PSHBM_FATAL : PSHBM_OK;
}

uint64_t pshbm_debug_tombstone_limit(uint64_t slots, uint64_t max_rows) { return tombstone_limit(slots, max_rows); }

int32_t pshbm_debug_part_min_keys(uint64_t keys) {
    part_set_min_keys((size_t)keys);
    return PSHBM_OK;
}

int32_t pshbm_debug_part_order(pshbm_table* t, uint32_t* items, size_t capacity, size_t* n_items,
                               uint32_t* partitions) {
    if (!t) return PSHBM_INVALID_ID;
    if (!items || !n_items || !partitions) return fail(t, PSHBM_ERROR, "part_order: null argument");
    DeviceGuard g(t->device);
    std::unique_lock<std::shared_mutex> lk(t->mu);
    *n_items = 0;
    *partitions = 0;
    if (!t->pt_order.p) return PSHBM_OK;
    HIP_TRY(t, hipDeviceSynchronize());
    uint32_t tag[2] = {0, 0};
    const uint32_t* d_order = static_cast<const uint32_t*>(t->pt_order.p);
    HIP_TRY(t, hipMemcpy(tag, d_order + PART_ORDER_TAG, sizeof tag, hipMemcpyDeviceToHost));
    if (tag[0] == 0) return PSHBM_OK;
    const size_t n = part_order_slots(tag[0]);
    if (n > capacity) return fail(t, PSHBM_ERROR, "part_order: %zu items, room for %zu", n, capacity);
    HIP_TRY(t, hipMemcpy(items, d_order, n * 4, hipMemcpyDeviceToHost));
    *n_items = n;
    *partitions = tag[0];
    return PSHBM_OK;
}

int32_t pshbm_debug_part_pass_capacity(uint32_t entries) {
    part_set_pass_capacity(entries);
    return PSHBM_OK;
}

int32_t pshbm_host_alloc(void** p, size_t bytes) {
    if (!p) return PSHBM_ERROR;
    hipError_t e = hipHostMalloc(p, bytes, hipHostMallocDefault);
    if (e == hipSuccess) return PSHBM_OK;
    return e == hipErrorOutOfMemory ? PSHBM_OUT_OF_MEMORY : PSHBM_ERROR;
}

int32_t pshbm_host_free(void* p) {
    return hipHostFree(p) == hipSuccess ? PSHBM_OK : PSHBM_ERROR;
}

}  // extern "C"
