// CPU oracle for the sparse-table Pull / Push / Store / Set / Load / Dump path.
//
// THIS IS TEST INFRASTRUCTURE, NOT PRODUCT CODE. It is a scalar restatement of the server-side
// operator loops of pico-ps over one shard, written to be read next to the reference. Only the
// tests, the smoke check and the benchmark's cpu_baseline leg may load it; the library under
// parameter-server_amd/ never does.
//
// Storage model: one shard = std::unordered_map<uint64_t, row index> plus a dense row slab, the
// model of UnorderedMapShardStorage (pico-ps/storage/KVShardStorage.h:102-188). Map semantics
// (find / insert-if-absent / upsert) follow lock_find / safe_insert / safe_set
// (KVShardStorage.h:786-814).
//
// Pinning status of each function (what its results are checked against, in tests/):
//   pso_pull, pso_set, pso_dump, pso_iterate, pso_load, pso_clear, pso_size
//       associative-container semantics; pinned by a brute-force std::map model, by the
//       invariants of the reference's test_sparse (pico-ps/test/ps_service_test.cpp:104-184)
//       and by its known answers (tests/golden/reference_known_answers.json), among them the
//       map contract's own unit tests (pico-ps/test/ps_pmem_test.cpp:110-193).
//   pso_aggregate, pso_push (SUM), pso_queue/pso_store (SUM)
//       pinned by the reference's integer test operator: pushing arg=key c times gives
//       sum = key*c, count = c (pico-ps/test/TestOps.h:98-117,171-172;
//       pico-ps/test/ps_pmem_test.cpp:401-439).
//   pso_for_each, pso_erase_if, pso_erase
//       pinned by the reference's test operators (pico-ps/test/TestOps.h:138-185: erase the odd
//       keys; count and sum every record) and the counts its service test asserts
//       (pico-ps/test/ps_service_test.cpp:158-166,176-184), and by a brute-force dict model.
//   pso_for_each_write
//       the loop is the reference's (ForEachOperator.h:277-359: every record, hook on a writable
//       value); the hook (affine map / clamp of a column range under a predicate) is this
//       repository's, the reference ships none that writes: PARITY UNPINNED BY THE REFERENCE,
//       pinned by an independent numpy model of the two formulas (tests/test_for_each_write.py).
//   pso_increment_size, pso_take_increment
//       which keys a push or store touched (the second storage the reference mirrors them into,
//       SparsePushOperator.h:253-266,394-407, read and emptied by IncrementStorage.h:29-36);
//       pinned by a dict-and-set model of those lines (tests/test_increment.py). The reference has
//       no test of its own for the increment.
//   Dense tables need nothing of their own here: a slice {id, slice_id} is the key
//       id << 24 | slice_id of the same functions; the reference's test_dense
//       (pico-ps/test/ps_service_test.cpp:241-409) is one of the known-answer scenarios.
//   SGD / ADAGRAD / FTRL arithmetic (apply_update below)
//       PARITY UNPINNED BY THE REFERENCE: pico-ps ships no optimizer (the update is the user
//       hook SparsePushOperator.h:448). The formulas are this repository's definition; they are
//       pinned by hand-computed single-key cases, a float64 re-evaluation and algebraic special
//       cases in tests/test_oracle_optimizers.py.
//   Initial weights of a new key (init_weight below, when init_range > 0)
//       PARITY UNPINNED BY THE REFERENCE: the value a pull or push inserts is the user hook
//       init_store_value (SparsePullOperator.h:307-310, SparsePushOperator.h:250-251), for which
//       pico-ps ships only zeros. The formula is this repository's; it is pinned by MurmurHash3's
//       published finalizer vectors, an integer-only Python restatement, the exact bounds and the
//       first two moments of the uniform distribution (tests/test_initial_weights.py).
//   Key partition (pso_partition, the PART_EQ / PART_NE terms of a predicate)
//       the shape is the reference's DefaultPartitioner<uint64_t> (pico-ps/common/Partitioner.h:43-61:
//       jump_consistent_hash(murmur_hash(key), n)); both functions live in pico-core, which the
//       reference tree does not hold: PARITY UNPINNED BY THE REFERENCE. Restated from their
//       publications and pinned by those: MurmurHash3's fmix64 (published finalizer vectors) and
//       the jump consistent hash of Lamping and Veach (arXiv:1406.2294; the test vectors of its widely
//       used Go port github.com/dgryski/go-jump, the paper's properties -- one bucket for n = 1,
//       keys only ever move to the new bucket when n grows, even spread -- and an integer-only
//       Python restatement) in tests/test_partitioner.py.
//   Capacity handling (PSO_OUT_OF_MEMORY, all-or-nothing per batch)
//       this repository's decision for a fixed-capacity table; the reference instead parks the
//       items in an overflow vector (SparsePushOperator.h:257-259). Documented, not pinned.

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <unordered_map>
#include <unordered_set>
#include <utility>
#include <vector>

namespace {

constexpr uint64_t KEY_EMPTY = 0xFFFFFFFFFFFFFFFFull;
constexpr uint64_t KEY_DELETED = 0xFFFFFFFFFFFFFFFEull;

enum { ST_OK = 0, ST_INVALID_CONFIG = 1, ST_OOM = 3, ST_ERROR = 10 };  // Status.h:15-29
enum { OPT_SUM = 0, OPT_SGD = 1, OPT_ADAGRAD = 2, OPT_FTRL = 3, OPT_USER = 4 };
enum { PULL_INSERT_ON_MISS = 1u, PUSH_NO_INSERT = 1u, LOAD_UNIQUE = 1u };
// Oracle-only push flag: sum duplicates in float64 and round once. This is not what the reference
// computes; it is the exactly rounded sum, against which tests judge which of two fp32 summation
// orders (the reference's sequential one, the kernels' tree) is closer for heavily repeated keys.
enum { PUSH_EXACT_AGGREGATION = 0x100u };

struct Config {
    uint32_t dim;
    int32_t optimizer;
    float lr, init_acc, alpha, beta, l1, l2;
    uint64_t capacity;
    int32_t read_only;
    int32_t track_increment;
    float init_range;
};

struct Oracle {
    Config c;
    uint32_t vf;  // floats per stored value
    std::unordered_map<uint64_t, uint32_t> map;
    std::vector<float> rows;         // size() * vf
    std::vector<uint64_t> row_keys;  // key of each row, slab order
    // sync-push queue (the MPSC queue of blocks, KVShardStorage.h:677-726), flattened
    std::vector<uint64_t> q_keys;
    std::vector<float> q_grads;
    // the increment: keys whose values a push or a store wrote since the last take (the reference
    // keeps copies of the values in a second storage, SparsePushOperator.h:253-266; the values are
    // read when the increment is taken, which gives the same records as long as nothing is pushed
    // in between)
    std::unordered_set<uint64_t> touched;
};

uint32_t value_floats(uint32_t dim, int32_t opt) {
    switch (opt) {
        case OPT_SUM:
        case OPT_SGD: return dim;
        case OPT_ADAGRAD: return 2 * dim;
        case OPT_FTRL: return 3 * dim;
        case OPT_USER: return 2 * dim;  // the rule shipped in parameter-server_amd/csrc/user_opt.h: one state block
    }
    return 0;
}

bool reserved(uint64_t k) { return k == KEY_EMPTY || k == KEY_DELETED; }

// MurmurHash3's 64-bit finalizer (Appleby, MurmurHash3.cpp, public domain).
uint64_t fmix64(uint64_t k) {
    k ^= k >> 33;
    k *= 0xff51afd7ed558ccdull;
    k ^= k >> 33;
    k *= 0xc4ceb9fe1a85ec53ull;
    k ^= k >> 33;
    return k;
}

// Weight j of a new key when the table draws initial weights: the top 24 bits of a hash of
// (key, column) as a number in [-1, 1) (exact in fp32), times the range (one rounding).
// DefaultPartitioner<uint64_t>::partition (pico-ps/common/Partitioner.h:36-38,47-54) with the
// published functions: fmix64, then the loop of Lamping and Veach's paper.
int32_t jump_partition(uint64_t key, int32_t n) {
    uint64_t k = fmix64(key);
    int64_t b = -1, j = 0;
    while (j < n) {
        b = j;
        k = k * 2862933555777941757ull + 1;
        j = (int64_t)((double)(b + 1) * ((double)(1ll << 31) / (double)((k >> 33) + 1)));
    }
    return (int32_t)b;
}

float init_weight(float range, uint64_t key, uint32_t j) {
    const uint64_t h = fmix64(key ^ ((uint64_t)(j + 1u) * 0x9E3779B97F4A7C15ull));
    const float unit = (float)(uint32_t)(h >> 40) * (1.0f / 8388608.0f) - 1.0f;
    return unit * range;
}

// value_type() of a key that a pull or push inserts: zero (or drawn) weights, fresh optimizer state.
void init_value(const Config& c, uint64_t key, float* v) {
    const uint32_t d = c.dim;
    for (uint32_t j = 0; j < d; ++j) v[j] = c.init_range != 0.0f ? init_weight(c.init_range, key, j) : 0.0f;
    if (c.optimizer == OPT_ADAGRAD)
        for (uint32_t j = 0; j < d; ++j) v[d + j] = c.init_acc;
    if (c.optimizer == OPT_FTRL)
        for (uint32_t j = 0; j < 2 * d; ++j) v[d + j] = 0.0f;
    if (c.optimizer == OPT_USER)  // momentum starts at rest
        for (uint32_t j = 0; j < d; ++j) v[d + j] = 0.0f;
}

// store_push_value (SparsePushOperator.h:448) for the optimizers this repository defines.
// Every operation is a separate fp32 rounding (compiled with -ffp-contract=off).
void apply_update(const Config& c, const float* g, float* v) {
    const uint32_t d = c.dim;
    switch (c.optimizer) {
        case OPT_SUM:  // TestPushOperator::store_push_value, pico-ps/test/TestOps.h:112-117
            for (uint32_t j = 0; j < d; ++j) v[j] = v[j] + g[j];
            break;
        case OPT_SGD:
            for (uint32_t j = 0; j < d; ++j) {
                float step = c.lr * g[j];
                v[j] = v[j] - step;
            }
            break;
        case OPT_ADAGRAD:
            for (uint32_t j = 0; j < d; ++j) {
                float gg = g[j] * g[j];
                float n = v[d + j] + gg;
                float num = c.lr * g[j];
                float step = num / sqrtf(n);
                v[d + j] = n;
                v[j] = v[j] - step;
            }
            break;
        case OPT_FTRL:
            for (uint32_t j = 0; j < d; ++j) {
                float w = v[j], z = v[d + j], n = v[2 * d + j];
                float gg = g[j] * g[j];
                float n_new = n + gg;
                float sq_new = sqrtf(n_new);
                float sigma = (sq_new - sqrtf(n)) / c.alpha;
                float sw = sigma * w;
                z = (z + g[j]) - sw;
                float w_new;
                if (fabsf(z) <= c.l1) {
                    w_new = 0.0f;
                } else {
                    float shrunk = z > 0.0f ? z - c.l1 : z + c.l1;
                    float denom = (c.beta + sq_new) / c.alpha + c.l2;
                    w_new = -shrunk / denom;
                }
                v[j] = w_new;
                v[d + j] = z;
                v[2 * d + j] = n_new;
            }
            break;
        case OPT_USER:  // mirror of the rule shipped as the library's user hook: SGD with momentum,
                        // v = beta * v + g; w = w - lr * v (heavy ball, Polyak 1964), one state block
            for (uint32_t j = 0; j < d; ++j) {
                float carried = c.beta * v[d + j];
                float vel = carried + g[j];
                float delta = c.lr * vel;
                v[d + j] = vel;
                v[j] = v[j] - delta;
            }
            break;
    }
}

uint32_t append_row(Oracle& o, uint64_t key) {
    uint32_t r = (uint32_t)o.row_keys.size();
    o.row_keys.push_back(key);
    o.rows.resize((size_t)(r + 1) * o.vf);
    o.map.emplace(key, r);
    return r;
}

// Duplicate aggregation of one client batch: generate_request_data,
// pico-ps/operator/SparsePushOperator.h:134-141. try_emplace -> init_push_value (zeros, :434-436)
// -> apply_push_arg adds each occurrence in input order. Unique keys come out in first-occurrence
// order (the reference's wire order is EasyHashMap bucket order, which fixes no value).
void aggregate(uint32_t dim, const uint64_t* keys, const float* grads, size_t n,
               std::vector<uint64_t>& ukeys, std::vector<float>& usum, bool exact = false) {
    std::unordered_map<uint64_t, size_t> whole_map;
    whole_map.reserve(n * 2);
    ukeys.clear();
    usum.clear();
    std::vector<double> dsum;  // exact mode only
    for (size_t i = 0; i < n; ++i) {
        auto rit = whole_map.try_emplace(keys[i], ukeys.size());
        if (rit.second) {
            ukeys.push_back(keys[i]);
            usum.resize(usum.size() + dim, 0.0f);
            if (exact) dsum.resize(dsum.size() + dim, 0.0);
        }
        const float* g = grads + i * dim;
        if (exact) {
            double* acc = &dsum[rit.first->second * dim];
            for (uint32_t j = 0; j < dim; ++j) acc[j] += (double)g[j];
        } else {
            float* acc = &usum[rit.first->second * dim];
            for (uint32_t j = 0; j < dim; ++j) acc[j] = acc[j] + g[j];
        }
    }
    if (exact)
        for (size_t k = 0; k < dsum.size(); ++k) usum[k] = (float)dsum[k];
}

// The per-item loop of apply_async_push_request, SparsePushOperator.h:245-268, over unique items.
int32_t apply_unique(Oracle& o, const std::vector<uint64_t>& ukeys, const std::vector<float>& usum,
                     uint32_t flags) {
    const bool insert = !(flags & PUSH_NO_INSERT);
    if (insert) {  // capacity pre-check: all-or-nothing
        uint64_t fresh = 0;
        for (uint64_t k : ukeys)
            if (!o.map.count(k)) ++fresh;
        if (o.map.size() + fresh > o.c.capacity) return ST_OOM;
    }
    for (size_t u = 0; u < ukeys.size(); ++u) {
        auto it = o.map.find(ukeys[u]);  // lock_find
        uint32_t r;
        if (it == o.map.end()) {
            if (!insert) continue;  // init_store_value returned false: item dropped (:250-251)
            r = append_row(o, ukeys[u]);
            init_value(o.c, ukeys[u], &o.rows[(size_t)r * o.vf]);
        } else {
            r = it->second;
        }
        apply_update(o.c, &usum[u * o.c.dim], &o.rows[(size_t)r * o.vf]);
        if (o.c.track_increment) o.touched.insert(ukeys[u]);  // safe_set(*incr_ht, ...), :253-266
    }
    return ST_OK;
}

}  // namespace

extern "C" {

struct pso_config {
    uint32_t dim;
    int32_t optimizer;
    float lr, init_acc, alpha, beta, l1, l2;
    uint64_t capacity;
    int32_t read_only;
    int32_t track_increment;
    float init_range;
};

float pso_init_weight(float range, uint64_t key, uint32_t column) { return init_weight(range, key, column); }
int32_t pso_partition(uint64_t key, int32_t n) { return n > 0 ? jump_partition(key, n) : -1; }

uint32_t pso_value_floats(uint32_t dim, int32_t opt) { return value_floats(dim, opt); }

// create_shard, KVShardStorage.h:910-925
int32_t pso_create(const pso_config* cfg, void** out) {
    if (!cfg || !out || cfg->dim == 0 || value_floats(cfg->dim, cfg->optimizer) == 0 ||
        cfg->capacity == 0 || !(cfg->init_range >= 0.0f && cfg->init_range <= 3.0e38f))
        return ST_INVALID_CONFIG;
    auto* o = new Oracle();
    o->c = Config{cfg->dim, cfg->optimizer, cfg->lr,  cfg->init_acc,  cfg->alpha,
                  cfg->beta, cfg->l1,       cfg->l2,  cfg->capacity,  cfg->read_only,
                  cfg->track_increment, cfg->init_range};
    o->vf = value_floats(cfg->dim, cfg->optimizer);
    *out = o;
    return ST_OK;
}

int32_t pso_destroy(void* h) {
    delete static_cast<Oracle*>(h);
    return ST_OK;
}

// SparseTablePullOperator::apply_request, SparsePullOperator.h:208-228 (one shard, one block).
int32_t pso_pull(void* h, const uint64_t* keys, size_t n, float* out_rows, uint8_t* hit,
                 uint32_t flags) {
    Oracle& o = *static_cast<Oracle*>(h);
    const uint32_t d = o.c.dim;
    const bool insert = (flags & PULL_INSERT_ON_MISS) && !o.c.read_only;  // :219
    for (size_t i = 0; i < n; ++i)
        if (reserved(keys[i])) return ST_ERROR;
    const uint32_t rows_at_entry = (uint32_t)o.row_keys.size();
    if (insert) {
        std::unordered_set<uint64_t> fresh;
        for (size_t i = 0; i < n; ++i)
            if (!o.map.count(keys[i])) fresh.insert(keys[i]);
        if (o.map.size() + fresh.size() > o.c.capacity) return ST_OOM;  // :245-253
    }
    std::vector<float> store_val(o.vf);
    for (size_t i = 0; i < n; ++i) {
        auto it = o.map.find(keys[i]);  // lock_find, :213
        const float* src;
        if (it != o.map.end()) {
            src = &o.rows[(size_t)it->second * o.vf];
            if (hit) hit[i] = it->second < rows_at_entry;  // mask against the table at entry
        } else {
            init_value(o.c, keys[i], store_val.data());  // init_store_value, :217
            src = store_val.data();
            if (hit) hit[i] = 0;
            if (insert) {  // safe_insert, :224
                uint32_t r = append_row(o, keys[i]);
                std::memcpy(&o.rows[(size_t)r * o.vf], store_val.data(), o.vf * sizeof(float));
            }
        }
        std::memcpy(out_rows + i * d, src, d * sizeof(float));  // fetch_pull_value + ps_serialize, :214,227
    }
    return ST_OK;
}

// Client-side aggregation alone (SparsePushOperator.h:134-141), for testing the reduction.
// ukeys/usum must hold n and n*dim entries; *n_unique receives the count.
int32_t pso_aggregate(uint32_t dim, const uint64_t* keys, const float* grads, size_t n,
                      uint64_t* ukeys, float* usum, size_t* n_unique) {
    std::vector<uint64_t> uk;
    std::vector<float> us;
    aggregate(dim, keys, grads, n, uk, us);
    std::copy(uk.begin(), uk.end(), ukeys);
    std::copy(us.begin(), us.end(), usum);
    *n_unique = uk.size();
    return ST_OK;
}

// One client batch end to end: aggregation (:134-141) then apply_async_push_request (:245-268).
int32_t pso_push(void* h, const uint64_t* keys, const float* grads, size_t n, uint32_t flags) {
    Oracle& o = *static_cast<Oracle*>(h);
    for (size_t i = 0; i < n; ++i)
        if (reserved(keys[i])) return ST_ERROR;
    std::vector<uint64_t> uk;
    std::vector<float> us;
    aggregate(o.c.dim, keys, grads, n, uk, us, (flags & PUSH_EXACT_AGGREGATION) != 0);
    return apply_unique(o, uk, us, flags);
}

// apply_sync_push_request, SparsePushOperator.h:299-316: the block is queued, nothing merged yet.
int32_t pso_queue(void* h, const uint64_t* keys, const float* grads, size_t n) {
    Oracle& o = *static_cast<Oracle*>(h);
    for (size_t i = 0; i < n; ++i)
        if (reserved(keys[i])) return ST_ERROR;
    o.q_keys.insert(o.q_keys.end(), keys, keys + n);
    o.q_grads.insert(o.q_grads.end(), grads, grads + n * o.c.dim);
    return ST_OK;
}

int32_t pso_queued(void* h, uint64_t* n) {
    *n = static_cast<Oracle*>(h)->q_keys.size();
    return ST_OK;
}

// apply_store_request, SparsePushOperator.h:374-409: blocks are drained in queue order, the first
// occurrence of a key becomes the accumulator and later ones are merged into it
// (merge_push_value = add), then every distinct key is applied once.
int32_t pso_store(void* h, uint32_t flags) {
    Oracle& o = *static_cast<Oracle*>(h);
    std::vector<uint64_t> uk;
    std::vector<float> us;
    aggregate(o.c.dim, o.q_keys.data(), o.q_grads.data(), o.q_keys.size(), uk, us);
    o.q_keys.clear();
    o.q_grads.clear();
    return apply_unique(o, uk, us, flags);
}

// DirectPushOperator::apply_async_push_request, SparsePushOperator.h:557-562: safe_set = upsert.
int32_t pso_set(void* h, const uint64_t* keys, const float* values, size_t n) {
    Oracle& o = *static_cast<Oracle*>(h);
    uint64_t fresh = 0;
    {
        std::unordered_set<uint64_t> seen;
        for (size_t i = 0; i < n; ++i) {
            if (reserved(keys[i])) return ST_ERROR;
            if (!o.map.count(keys[i]) && seen.insert(keys[i]).second) ++fresh;
        }
    }
    if (o.map.size() + fresh > o.c.capacity) return ST_OOM;  // :568-573
    for (size_t i = 0; i < n; ++i) {
        auto it = o.map.find(keys[i]);
        uint32_t r = it == o.map.end() ? append_row(o, keys[i]) : it->second;
        std::memcpy(&o.rows[(size_t)r * o.vf], values + i * o.vf, o.vf * sizeof(float));
    }
    return ST_OK;
}

// BaseKVTextFileLoadOperator::restore, LoadOperator.h:164-213, after the file is decoded into
// records {uint64 key; float value[vf]}. With LOAD_UNIQUE a present key fails (SCHECK, :194,210).
int32_t pso_load(void* h, const void* records, size_t n, uint32_t flags) {
    Oracle& o = *static_cast<Oracle*>(h);
    const size_t rec = 8 + (size_t)o.vf * 4;
    const char* p = static_cast<const char*>(records);
    bool skipped = false;  // a record with a reserved key is left out and the load reports an error
    for (size_t i = 0; i < n; ++i) {
        uint64_t key;
        std::memcpy(&key, p + i * rec, 8);
        if (reserved(key)) {
            skipped = true;
            continue;
        }
        auto it = o.map.find(key);
        if (it != o.map.end() && (flags & LOAD_UNIQUE)) return ST_ERROR;
        if (it == o.map.end() && o.map.size() + 1 > o.c.capacity) return ST_OOM;
        uint32_t r = it == o.map.end() ? append_row(o, key) : it->second;
        std::memcpy(&o.rows[(size_t)r * o.vf], p + i * rec + 8, (size_t)o.vf * 4);
    }
    return skipped ? ST_ERROR : ST_OK;
}

// KVShardIterator::iterate_batch_as_binary_archive, KVShardStorage.h:64-87: records
// [offset, offset+batch) of the shard in iteration order (here: slab order).
int32_t pso_iterate(void* h, size_t offset, size_t batch, void* records, size_t* n_out) {
    Oracle& o = *static_cast<Oracle*>(h);
    const size_t rec = 8 + (size_t)o.vf * 4;
    char* p = static_cast<char*>(records);
    size_t end = std::min(offset + batch, o.row_keys.size());
    size_t w = 0;
    for (size_t r = offset; r < end; ++r, ++w) {
        std::memcpy(p + w * rec, &o.row_keys[r], 8);
        std::memcpy(p + w * rec + 8, &o.rows[r * o.vf], (size_t)o.vf * 4);
    }
    *n_out = w;
    return ST_OK;
}

// BaseKVTextFileDumpOperator::apply_request, DumpOperator.h:163-174: every (key, value) once.
int32_t pso_dump(void* h, void* records, size_t capacity_records, size_t* n_out) {
    Oracle& o = *static_cast<Oracle*>(h);
    if (capacity_records < o.row_keys.size()) return ST_ERROR;
    return pso_iterate(h, 0, o.row_keys.size(), records, n_out);
}

// ---- for-each / erase-if -------------------------------------------------------------------
// The hooks the reference leaves to the application (for_each, erase_if) in the declarative form
// the device library evaluates: up to four comparisons on the key or on value columns, all of
// which must hold. Layout identical to pshbm_term / pshbm_predicate.
struct pso_term {
    int32_t column;  // -1 = the key
    int32_t cmp;     // 0 LT, 1 LE, 2 GT, 3 GE, 4 EQ, 5 NE, 6 MOD_EQ (key % u == u2),
                     // 7 PART_EQ / 8 PART_NE (the key's partition among u is / is not u2)
    float f;
    uint32_t reserved;
    uint64_t u, u2;
};
struct pso_predicate {
    uint32_t struct_size;
    uint32_t n_terms;
    pso_term term[4];
};

static bool holds(const pso_predicate* p, uint64_t key, const float* v) {
    if (!p) return true;
    for (uint32_t i = 0; i < p->n_terms; ++i) {
        const pso_term& t = p->term[i];
        bool r = false;
        if (t.column < 0) {
            switch (t.cmp) {
                case 0: r = key < t.u; break;
                case 1: r = key <= t.u; break;
                case 2: r = key > t.u; break;
                case 3: r = key >= t.u; break;
                case 4: r = key == t.u; break;
                case 5: r = key != t.u; break;
                case 6: r = t.u != 0 && key % t.u == t.u2; break;
                case 7: r = t.u != 0 && (uint64_t)jump_partition(key, (int32_t)t.u) == t.u2; break;
                case 8: r = t.u != 0 && (uint64_t)jump_partition(key, (int32_t)t.u) != t.u2; break;
            }
        } else {
            const float x = v[t.column];
            switch (t.cmp) {
                case 0: r = x < t.f; break;
                case 1: r = x <= t.f; break;
                case 2: r = x > t.f; break;
                case 3: r = x >= t.f; break;
                case 4: r = x == t.f; break;
                case 5: r = x != t.f; break;
            }
        }
        if (!r) return false;
    }
    return true;
}

// safe_erase (KVShardStorage.h:827-834) on the slab model: the last row takes the erased row's
// place, so the slab stays dense; iteration order after an erase is unspecified, as in the reference.
static void erase_row(Oracle& o, uint32_t r) {
    const uint32_t last = (uint32_t)o.row_keys.size() - 1;
    o.touched.erase(o.row_keys[r]);
    o.map.erase(o.row_keys[r]);
    if (r != last) {
        o.row_keys[r] = o.row_keys[last];
        std::memcpy(&o.rows[(size_t)r * o.vf], &o.rows[(size_t)last * o.vf], (size_t)o.vf * 4);
        o.map[o.row_keys[r]] = r;
    }
    o.row_keys.pop_back();
    o.rows.resize((size_t)last * o.vf);
}

// SparseTableForEachReadOperator::apply_request, ForEachOperator.h:180-190, with the hook
// "result = {1, value}" and merge_result = add (the shape of TestForEachOperator, TestOps.h:159-185):
// *count = records that satisfy the predicate, sums[c] = sum of value column c over them.
int32_t pso_for_each(void* h, const pso_predicate* where, uint64_t* count, double* sums) {
    Oracle& o = *static_cast<Oracle*>(h);
    uint64_t n = 0;
    if (sums)
        for (uint32_t c = 0; c < o.vf; ++c) sums[c] = 0.0;
    for (size_t r = 0; r < o.row_keys.size(); ++r) {
        const float* v = &o.rows[r * o.vf];
        if (!holds(where, o.row_keys[r], v)) continue;
        ++n;
        if (sums)
            for (uint32_t c = 0; c < o.vf; ++c) sums[c] += (double)v[c];
    }
    *count = n;
    return ST_OK;
}

// SparseTableForEachWriteOperator::apply_request, ForEachOperator.h:277-359, with the hook "rewrite
// columns [first, first + n) of the value": op 0: a * v + b (two roundings), op 1: clamp to [a, b].
// The predicate sees the value before the rewrite. *count = records rewritten.
struct pso_update {
    uint32_t struct_size;
    int32_t op;
    uint32_t first_column, n_columns;
    float a, b;
};
int32_t pso_for_each_write(void* h, const pso_predicate* where, const pso_update* what, uint64_t* count) {
    Oracle& o = *static_cast<Oracle*>(h);
    if (o.c.read_only) return ST_ERROR;
    if (!what || (uint64_t)what->first_column + what->n_columns > o.vf || what->op < 0 || what->op > 1)
        return ST_INVALID_CONFIG;
    uint64_t n = 0;
    for (size_t r = 0; r < o.row_keys.size(); ++r) {
        float* v = &o.rows[r * o.vf];
        if (!holds(where, o.row_keys[r], v)) continue;
        ++n;
        for (uint32_t c = what->first_column; c < what->first_column + what->n_columns; ++c) {
            if (what->op == 0) {
                const float p = what->a * v[c];
                v[c] = p + what->b;
            } else {
                v[c] = std::fmin(std::fmax(v[c], what->a), what->b);
            }
        }
        if (o.c.track_increment) o.touched.insert(o.row_keys[r]);
    }
    if (count) *count = n;
    return ST_OK;
}

// SparseTableEraseIfOperator::apply_request, EraseIfOperator.h:38-47.
int32_t pso_erase_if(void* h, const pso_predicate* where, uint64_t* erased) {
    Oracle& o = *static_cast<Oracle*>(h);
    if (o.c.read_only) return ST_ERROR;
    uint64_t n = 0;
    for (size_t r = 0; r < o.row_keys.size();) {
        if (holds(where, o.row_keys[r], &o.rows[r * o.vf])) {
            erase_row(o, (uint32_t)r);  // the row that moved in is examined next
            ++n;
        } else {
            ++r;
        }
    }
    if (erased) *erased = n;
    return ST_OK;
}

// erase of chosen keys: what an erase_if hook evaluated outside the storage comes down to.
int32_t pso_erase(void* h, const uint64_t* keys, size_t n, uint64_t* erased) {
    Oracle& o = *static_cast<Oracle*>(h);
    if (o.c.read_only) return ST_ERROR;
    uint64_t gone = 0;
    for (size_t i = 0; i < n; ++i) {
        if (reserved(keys[i])) return ST_ERROR;
        auto it = o.map.find(keys[i]);
        if (it == o.map.end()) continue;
        erase_row(o, it->second);
        ++gone;
    }
    if (erased) *erased = gone;
    return ST_OK;
}

// The hyperparameters belong to the push operator (Operator.h:53-57); a new operator brings new ones.
int32_t pso_set_hyperparameters(void* h, float lr, float init_acc, float alpha, float beta, float l1,
                                float l2) {
    Oracle& o = *static_cast<Oracle*>(h);
    if (o.c.optimizer == OPT_FTRL && !(alpha > 0.0f)) return ST_INVALID_CONFIG;
    o.c.lr = lr;
    o.c.init_acc = init_acc;
    o.c.alpha = alpha;
    o.c.beta = beta;
    o.c.l1 = l1;
    o.c.l2 = l2;
    return ST_OK;
}

// A growing hash map rehashes by itself (safe_insert, KVShardStorage.h:791-801); the fixed-capacity
// model only raises its limit.
int32_t pso_reserve(void* h, uint64_t capacity) {
    Oracle& o = *static_cast<Oracle*>(h);
    if (capacity > 0xFFFFFFF0ull) return ST_INVALID_CONFIG;
    if (capacity > o.c.capacity) o.c.capacity = capacity;
    return ST_OK;
}

// IncrementStorage::read_storage + the sync operator's walk of it (service/IncrementStorage.h:29-36,
// operator/SyncOperator.h:185-266): the {key, value} records of the keys pushes wrote since the
// last take, then the increment is empty. Too little room: ST_ERROR, *n_out = records needed.
int32_t pso_increment_size(void* h, uint64_t* n) {
    *n = static_cast<Oracle*>(h)->touched.size();
    return ST_OK;
}
int32_t pso_take_increment(void* h, void* records, size_t capacity_records, size_t* n_out) {
    Oracle& o = *static_cast<Oracle*>(h);
    *n_out = o.touched.size();
    if (o.touched.size() > capacity_records) return ST_ERROR;
    const size_t rec = 8 + (size_t)o.vf * 4;
    char* p = static_cast<char*>(records);
    size_t w = 0;
    for (uint64_t k : o.touched) {
        const uint32_t r = o.map.at(k);
        std::memcpy(p + w * rec, &k, 8);
        std::memcpy(p + w * rec + 8, &o.rows[(size_t)r * o.vf], (size_t)o.vf * 4);
        ++w;
    }
    o.touched.clear();
    return ST_OK;
}

// KVShardStorage::clear, KVShardStorage.h:902-908
int32_t pso_clear(void* h) {
    Oracle& o = *static_cast<Oracle*>(h);
    o.map.clear();
    o.rows.clear();
    o.row_keys.clear();
    o.touched.clear();
    return ST_OK;
}

// shard_size, KVShardStorage.h:927-935
int32_t pso_size(void* h, uint64_t* n) {
    *n = static_cast<Oracle*>(h)->map.size();
    return ST_OK;
}

}  // extern "C"
