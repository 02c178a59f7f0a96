// Host-side mirror of the pico-ps operator interface for the sparse-table path, on top of the
// C ABI of include/pshbm.h. Each class stands where the reference class of the same role stands
// and keeps its method names, argument order and error behaviour; only the body differs: instead
// of walking a hash map key by key, it hands the decoded block to the HBM table.
//
//   HbmShardStorage        <- KVShardStorage / PoolHashMapShardStorage (storage/KVShardStorage.h:22-49, 844-952)
//   HbmStorageOperator     <- ShardStorageOperator                     (operator/StorageOperator.h:78-158)
//   HbmSyncOperator        <- KVSyncOperator                           (operator/SyncOperator.h:102-266)
//   HbmSparsePullOperator  <- SparseTablePullOperator::apply_request   (operator/SparsePullOperator.h:156-254)
//   HbmSparsePushOperator  <- SparseTablePushOperator server halves    (operator/SparsePushOperator.h:197-416)
//   HbmDirectPushOperator  <- DirectPushOperator                       (operator/SparsePushOperator.h:520-574)
//   HbmDensePushOperator   <- DenseTablePushOperator server halves     (operator/DensePushOperator.h:137-316)
//   HbmDensePullOperator   <- DenseTablePullOperator::apply_request    (operator/DensePullOperator.h:118-181)
//   HbmDumpOperator        <- BaseKVTextFileDumpOperator::apply_request (operator/DumpOperator.h:137-183)
//   HbmLoadOperator        <- BaseKVTextFileLoadOperator::restore      (operator/LoadOperator.h:164-213)
//   HbmForEachOperator     <- SparseTableForEachReadOperator           (operator/ForEachOperator.h:150-233)
//   HbmEraseIfOperator     <- SparseTableEraseIfOperator               (operator/EraseIfOperator.h:18-58)
//   HbmShuffleOperator     <- ShufflePushItemsGenerator / apply_purge_request (operator/UpdateContextOperator.h:143-297)
//   HbmRestoreOperator     <- coordinated restore                      (operator/RestoreOperator.h:100-151)
//
// The client halves (generate_request, apply_response, ...) are not here: they run in the
// application process and are inherited unchanged from the reference's templates.
#pragma once

#include <algorithm>
#include <functional>
#include <memory>
#include <mutex>
#include <type_traits>
#include <unordered_map>

#include "../../include/pshbm.h"
#include "standin.h"

namespace pshbm_host {

// op_config keys of an HBM table: dim, optimizer (sum|sgd|adagrad|ftrl|user), lr, init_acc, alpha, beta,
// l1, l2, hbm_table.expected_max_items, hbm_table.grow_limit, hbm_table.max_load_factor,
// hbm_table.max_batch, hbm_table.track_increment, hbm_table.init_range, read_only, device. The learning rate lives in the operator config, as pico-ps/operator/Operator.h:55 expects.
inline pshbm_config table_config(const Configure& c) {
    pshbm_config cfg{};
    cfg.struct_size = sizeof(cfg);
    cfg.device = (int32_t)c.number("device", 0);
    cfg.dim = (uint32_t)c.number("dim", 0);
    const std::string opt = c.str("optimizer", "sum");
    cfg.optimizer = opt == "sgd" ? PSHBM_OPT_SGD : opt == "adagrad" ? PSHBM_OPT_ADAGRAD
                  : opt == "ftrl" ? PSHBM_OPT_FTRL : opt == "user" ? PSHBM_OPT_USER
                  : opt == "sum" ? PSHBM_OPT_SUM : -1;
    cfg.lr = (float)c.number("lr", 0.0);
    cfg.init_acc = (float)c.number("init_acc", 0.0);
    cfg.alpha = (float)c.number("alpha", 0.0);
    cfg.beta = (float)c.number("beta", 0.0);
    cfg.l1 = (float)c.number("l1", 0.0);
    cfg.l2 = (float)c.number("l2", 0.0);
    cfg.expected_max_items = (uint64_t)c.number("hbm_table.expected_max_items", 1 << 20);
    cfg.max_load_factor = (float)c.number("hbm_table.max_load_factor", 0.0);
    cfg.max_batch = (uint64_t)c.number("hbm_table.max_batch", 0);
    cfg.read_only = (int32_t)c.number("read_only", 0);
    cfg.track_increment = (int32_t)c.number("hbm_table.track_increment", 0);
    cfg.init_range = (float)c.number("hbm_table.init_range", 0.0);
    return cfg;
}

// The server's memory limit, for the device: what ShardStorageMemory::singleton().initialize(soft,
// hard) is for the host's memory (pico-ps/storage/Storage.cpp:93-98). Past `hard_limit` bytes held by
// all tables on `device`, creating a shard, growing one or sizing a workspace fails with
// OUT_OF_MEMORY, which the operators answer as Status::OOM; 0 lifts the limit.
inline void initialize_device_memory(int32_t device, uint64_t hard_limit) {
    PSHBM_SCHECK(pshbm_set_memory_limit(device, hard_limit) == PSHBM_OK, "bad device");
}

// One pshbm_table per local shard id, the way PmemHashMapShardStorage keeps one handle per shard
// (storage/DCPmemory.h:400-442). HBM is volatile: need_remote_restore() is true.
class HbmShardStorage : public Storage {
public:
    HbmShardStorage(const std::set<int32_t>& shard_ids, const Configure& config) : _config(config) {
        for (int32_t id : shard_ids) PSHBM_SCHECK(create_shard(id), "create_shard failed: " + _error);
    }
    ~HbmShardStorage() override {
        for (auto& p : _shards) pshbm_destroy(p.second);
    }
    HbmShardStorage(const HbmShardStorage&) = delete;
    HbmShardStorage& operator=(const HbmShardStorage&) = delete;

    bool need_remote_restore() override { return true; }
    pshbm_table* get(int32_t shard_id) {
        auto it = _shards.find(shard_id);
        return it == _shards.end() ? nullptr : it->second;
    }
    bool create_shard(int32_t shard_id) {  // KVShardStorage.h:910-925
        if (_shards.count(shard_id)) return false;
        pshbm_config cfg = table_config(_config);
        pshbm_table* t = nullptr;
        int32_t st = pshbm_create(&cfg, &t);
        if (st != PSHBM_OK) {
            _error = pshbm_last_error(nullptr);
            return false;
        }
        _shards[shard_id] = t;
        _locks[shard_id];  // (map nodes stay where they are: the mutex may be held while other shards come and go)
        _capacity[shard_id] = cfg.expected_max_items;
        _vf = pshbm_value_floats(cfg.dim, cfg.optimizer);
        _dim = cfg.dim;
        return true;
    }
    bool erase_shard(int32_t shard_id) {
        auto it = _shards.find(shard_id);
        if (it == _shards.end()) return false;
        pshbm_destroy(it->second);
        _shards.erase(it);
        return true;
    }
    // The exclusive side of the shard lock that the reference's push and store take
    // (SparsePushOperator.h:220,343: shard.lock()): held by an operator from the moment it hands its
    // hyperparameters to the shard's table until its block is applied (and the table grown, if it
    // had to be), so that server threads pushing to one shard neither race on this object's
    // bookkeeping nor apply a block with another operator's hyperparameters. The table's own
    // calls are thread-safe without it.
    std::unique_lock<std::mutex> lock_shard(int32_t shard_id) { return std::unique_lock<std::mutex>(_locks.at(shard_id)); }

    // A hash map of the reference grows inside the insert that needs the room (safe_insert,
    // KVShardStorage.h:791-801) until the memory limit makes it unhealthy; a table grows when an
    // operator finds it full: twice the capacity at a time, up to op_config
    // `hbm_table.grow_limit` keys (0, the default: never). False = no room to be had. The caller
    // holds lock_shard(shard_id).
    bool grow(int32_t shard_id) {
        const uint64_t limit = (uint64_t)_config.number("hbm_table.grow_limit", 0);
        pshbm_table* t = get(shard_id);
        if (!t || _capacity[shard_id] >= limit) return false;
        const uint64_t want = std::min<uint64_t>(limit, _capacity[shard_id] * 2);
        if (pshbm_reserve(t, want) != PSHBM_OK) {
            _error = pshbm_last_error(t);
            return false;
        }
        _capacity[shard_id] = want;
        return true;
    }
    // The hyperparameters of the push operator that is about to touch the shard (they live in the
    // operator's config, pico-ps/operator/Operator.h:53-57): handed to the table when they differ
    // from the ones it has. Operators with different hyperparameters must not push to one table at
    // the same time (the reference advises against changing a registered operator's config at all).
    // The caller holds lock_shard(shard_id).
    void use_hyperparameters(int32_t shard_id, const pshbm_hyperparameters& hp) {
        auto it = _hp.find(shard_id);
        if (it != _hp.end() && std::memcmp(&it->second, &hp, sizeof hp) == 0) return;
        PSHBM_SCHECK(pshbm_set_hyperparameters(get(shard_id), &hp) == PSHBM_OK,
                     std::string("bad hyperparameters: ") + pshbm_last_error(nullptr));
        _hp[shard_id] = hp;
    }
    void clear() {  // KVShardStorage.h:902-908: every shard emptied, the shards stay
        for (auto& p : _shards) pshbm_clear(p.second);
    }
    std::vector<int32_t> shard_list() const {
        std::vector<int32_t> ids;
        for (auto& p : _shards) ids.push_back(p.first);
        return ids;
    }
    size_t shard_size(int32_t shard_id) {  // :927-935
        uint64_t n = 0;
        pshbm_size(_shards.at(shard_id), &n);
        return n;
    }
    size_t shard_memory_usage(int32_t shard_id) {  // :937-946
        uint64_t n = 0;
        pshbm_memory_usage(_shards.at(shard_id), &n);
        return n;
    }
    // KVShardIterator::iterate_batch_as_binary_archive (:64-87): records [offset, offset+batch) of a
    // shard as {uint64 key, value} pairs appended to `ar`; returns how many (fewer than batch = end).
    size_t iterate_batch_as_binary_archive(int32_t shard_id, size_t offset, size_t batch, BinaryArchive& ar) {
        std::vector<char> rec(batch * record_bytes());
        size_t got = 0;
        int32_t st = pshbm_iterate(_shards.at(shard_id), offset, batch, rec.data(), &got);
        PSHBM_SCHECK(st == PSHBM_OK, "iterate failed");
        ar.write_raw(rec.data(), got * record_bytes());
        return got;
    }
    uint32_t dim() const { return _dim; }
    uint32_t value_floats() const { return _vf; }
    size_t record_bytes() const { return 8 + (size_t)_vf * 4; }
    const std::string& error() const { return _error; }

private:
    Configure _config;
    std::map<int32_t, pshbm_table*> _shards;
    std::map<int32_t, std::mutex> _locks;
    std::map<int32_t, uint64_t> _capacity;  // keys each shard's table holds at most
    std::map<int32_t, pshbm_hyperparameters> _hp;  // what each shard's table was last given
    uint32_t _dim = 0, _vf = 0;
    std::string _error;
};

// Marker for the delta storage of the sync path: the queue of blocks (SizeMpscQueueShardStorage,
// KVShardStorage.h:677-726) lives inside each shard's table.
class HbmDeltaStorage : public Storage {};

class HbmStorageOperator {
public:
    explicit HbmStorageOperator(const Configure& config) : _config(config) {}
    std::unique_ptr<Storage> create_storage(RuntimeInfo& rt, int32_t /*storage_id*/) {  // StorageOperator.h:106-109
        return std::make_unique<HbmShardStorage>(rt.local_shards(), _config);
    }
    void clear_storage(Storage* st) { static_cast<HbmShardStorage*>(st)->clear(); }  // :111-113
    void apply_query_info_request(RuntimeInfo& rt, PSRequest& req, Storage* storage, PSResponse& resp_ret) {  // :123-141
        std::vector<StorageStatisticInfo> info;
        auto* st = static_cast<HbmShardStorage*>(storage);
        for (int32_t shard_id : rt.local_shards())
            info.push_back({rt.node_id(), shard_id, st->shard_size(shard_id), st->shard_memory_usage(shard_id)});
        PSResponse resp(req);
        resp << info;
        resp_ret = std::move(resp);
    }

private:
    Configure _config;
};

// Server half of the sparse pull. Request: i32 shards_num, i32 merge_num; per shard {i32 shard_id;
// per merged request {i32 n; if n: one lazy block of n raw uint64 keys}} (SparsePullOperator.h:132-147).
// Response: i32 shards_num; the shard ids; then merge_num lazy blocks, block i holding the pulled
// values of merged request i over all shards, in request order (:170-171,183,227,238-244).
class HbmSparsePullOperator {
public:
    explicit HbmSparsePullOperator(const Configure& config)
        : _read_only(config.number("read_only", 0) != 0),
          _insert_on_miss(config.number("pull_insert_on_miss", 0) != 0) {}

    void apply_request(RuntimeInfo& rt, PSRequest& req, Storage* storage, PSResponse& resp) {
        int32_t shards_num, merge_num;
        req >> shards_num >> merge_num;
        std::vector<std::vector<char>> values_ars(merge_num);
        resp = PSResponse(req);
        resp << shards_num;
        bool healthy = true;
        std::string why;
        auto& st = *static_cast<HbmShardStorage*>(storage);
        const size_t row_bytes = (size_t)st.dim() * 4;
        const uint32_t flags = (_insert_on_miss && !_read_only) ? PSHBM_PULL_INSERT_ON_MISS : 0u;  // :219
        while (shards_num--) {
            int32_t shard_id;
            req >> shard_id;
            resp << shard_id;
            PSHBM_SCHECK(rt.local_shards().count(shard_id) != 0, "Bad Request: invalid shard_id");  // :185
            pshbm_table* t = st.get(shard_id);
            for (int i = 0; i < merge_num; ++i) {
                int32_t shard_keys_num;
                req >> shard_keys_num;
                if (shard_keys_num == 0) continue;  // :203-205: no block follows an empty count
                std::vector<char> keys_ar;
                ps_deserialize(req.lazy(), keys_ar);
                PSHBM_SCHECK(keys_ar.size() == (size_t)shard_keys_num * 8, "key block size mismatch");
                std::vector<char>& out = values_ars[i];
                const size_t at = out.size();
                out.resize(at + (size_t)shard_keys_num * row_bytes);
                int32_t rc = pshbm_pull(t, reinterpret_cast<const uint64_t*>(keys_ar.data()), shard_keys_num,
                                        reinterpret_cast<float*>(out.data() + at), nullptr, flags);
                if (rc != PSHBM_OK) {
                    healthy = false;
                    why = pshbm_last_error(t);
                }
            }
        }
        if (healthy) {
            for (auto& values_ar : values_ars) ps_serialize(resp.lazy(), std::move(values_ar));
        } else {  // :245-253: the whole response is replaced
            resp = PSResponse(req);
            resp.rpc_response().set_error_code(RpcErrorCodeType::ELOGICERROR);
            resp << Status::OOM("PServer OOM during pull: " + why);
        }
    }

private:
    bool _read_only, _insert_on_miss;
};

// Server halves of the sparse push. A push block is n raw std::pair<KEY, PUSH_VALUE> records, here
// {uint64 key, dim floats} (SparsePushOperator.h:164-179, 245-247).
// lr, init_acc, alpha, beta, l1, l2 of an operator's config, if it names any of them
inline bool operator_hyperparameters(const Configure& c, pshbm_hyperparameters* hp) {
    const pshbm_config cfg = table_config(c);
    *hp = pshbm_hyperparameters{sizeof(pshbm_hyperparameters), cfg.lr, cfg.init_acc, cfg.alpha, cfg.beta, cfg.l1, cfg.l2};
    for (const char* k : {"lr", "init_acc", "alpha", "beta", "l1", "l2"})
        if (c.has(k)) return true;
    return false;
}

class HbmSparsePushOperator {
public:
    explicit HbmSparsePushOperator(const Configure& config) : _has_hp(operator_hyperparameters(config, &_hp)) {}

    // apply_async_push_request, SparsePushOperator.h:197-276. Differences, both documented in
    // include/pshbm.h: equal keys inside one block are summed (the reference's client never sends
    // them); a block that does not fit is refused whole and the response carries Status::OOM (the
    // reference parks the items in the shard's overflow vector and answers OK, :257-259, :274-275).
    void apply_async_push_request(RuntimeInfo& rt, PSRequest& req, Storage* storage, Storage* /*incr_storage*/,
                                  PSResponse& resp) {
        Status status;
        auto& st = *static_cast<HbmShardStorage*>(storage);
        for_each_block(rt, req, storage, [&](int32_t shard_id, pshbm_table* t, const std::vector<char>& block, int32_t n, size_t stride) {
            auto lk = st.lock_shard(shard_id);  // shard.lock(), :220
            if (_has_hp) st.use_hyperparameters(shard_id, _hp);
            int32_t rc = pshbm_push_pairs(t, block.data(), n, stride, 0);
            while (rc == PSHBM_OUT_OF_MEMORY && st.grow(shard_id)) rc = pshbm_push_pairs(t, block.data(), n, stride, 0);
            if (rc == PSHBM_OUT_OF_MEMORY) status = Status::OOM(pshbm_last_error(t));
            else if (rc != PSHBM_OK) status = Status::Error(pshbm_last_error(t));
        });
        PSHBM_SCHECK(req.archive().is_exhausted(), "request not exhausted");  // :272
        resp = PSResponse(req);
        if (!status.ok()) resp.rpc_response().set_error_code(RpcErrorCodeType::ELOGICERROR);
        resp << status;
    }

    // apply_sync_push_request, :278-320: blocks are queued, nothing is merged or applied yet.
    void apply_sync_push_request(RuntimeInfo& rt, PSRequest& req, Storage* storage, PSResponse& resp) {
        Status status;
        for_each_block(rt, req, storage, [&](int32_t, pshbm_table* t, const std::vector<char>& block, int32_t n, size_t stride) {
            if (pshbm_queue_pairs(t, block.data(), n, stride) != PSHBM_OK) status = Status::Error(pshbm_last_error(t));
        });
        resp = PSResponse(req);
        resp << status;
    }

    // apply_store_request, :322-416: acknowledge first (:370-372), then merge and apply.
    void apply_store_request(RuntimeInfo& rt, PSRequest& req, Storage* delta_storage, Storage* storage,
                             Storage* /*incr_storage*/, std::function<void(PSResponse&&)> send_response) {
        int32_t shard_id;
        req >> shard_id;
        PSHBM_SCHECK(req.archive().is_exhausted(), "request not exhausted");
        PSHBM_SCHECK(rt.local_shards().count(shard_id), "Bad Request: invalid shard_id");
        PSResponse resp(req);
        resp << Status();
        send_response(std::move(resp));
        if (delta_storage == nullptr) return;  // :336-341
        auto lk = static_cast<HbmShardStorage*>(storage)->lock_shard(shard_id);  // shard.lock(), :343
        if (_has_hp) static_cast<HbmShardStorage*>(storage)->use_hyperparameters(shard_id, _hp);
        pshbm_store(static_cast<HbmShardStorage*>(storage)->get(shard_id), 0);
    }

    std::unique_ptr<Storage> create_delta_storage(RuntimeInfo&) { return std::make_unique<HbmDeltaStorage>(); }  // :425-427

private:
    pshbm_hyperparameters _hp{};
    bool _has_hp;

    template <class F>
    static void for_each_block(RuntimeInfo& rt, PSRequest& req, Storage* storage, F&& f) {
        int32_t shards_num, merge_num;
        req >> shards_num >> merge_num;
        auto& st = *static_cast<HbmShardStorage*>(storage);
        const size_t stride = 8 + (size_t)st.dim() * 4;
        while (shards_num--) {
            int32_t shard_id;
            req >> shard_id;
            PSHBM_SCHECK(rt.local_shards().count(shard_id) != 0, "Bad Request: invalid shard_id");
            pshbm_table* t = st.get(shard_id);
            for (int i = 0; i < merge_num; ++i) {
                int32_t shard_items_num;
                req >> shard_items_num;
                if (shard_items_num == 0) continue;
                std::vector<char> ar;
                ps_deserialize(req.lazy(), ar);
                PSHBM_SCHECK(ar.size() == (size_t)shard_items_num * stride, "push block size mismatch");
                f(shard_id, t, ar, shard_items_num, stride);
            }
        }
    }
};

// Of the n records {uint64 key, value} of `rec` bytes each, in place: the last record of every key,
// in the order of those last occurrences. Returns how many are left. (Blocks without a repeated
// key -- the normal case -- are left as they are after one pass over the keys.)
inline size_t keep_last_of_each_key(char* records, size_t n, size_t rec) {
    std::unordered_map<uint64_t, size_t> last;
    last.reserve(n * 2);
    bool repeats = false;
    for (size_t i = 0; i < n; ++i) {
        uint64_t k;
        std::memcpy(&k, records + i * rec, 8);
        auto it = last.find(k);
        if (it == last.end()) last.emplace(k, i);
        else {
            it->second = i;
            repeats = true;
        }
    }
    if (!repeats) return n;
    size_t out = 0;
    for (size_t i = 0; i < n; ++i) {
        uint64_t k;
        std::memcpy(&k, records + i * rec, 8);
        if (last[k] != i) continue;
        if (out != i) std::memmove(records + out * rec, records + i * rec, rec);
        ++out;
    }
    return out;
}

// DirectPushOperator::apply_async_push_request, SparsePushOperator.h:520-574: every item is
// {key, whole value}; ht[key] = value. OOM -> ELOGICERROR + Status::OOM (:568-573).
class HbmDirectPushOperator {
public:
    explicit HbmDirectPushOperator(const Configure&) {}
    void apply_async_push_request(RuntimeInfo& rt, PSRequest& req, Storage* storage, Storage*, PSResponse& resp) {
        resp = PSResponse(req);
        int32_t shards_num, merge_num;
        req >> shards_num >> merge_num;
        bool healthy = true;
        auto& st = *static_cast<HbmShardStorage*>(storage);
        while (shards_num--) {
            int32_t shard_id;
            req >> shard_id;
            PSHBM_SCHECK(rt.local_shards().count(shard_id) != 0, "Bad Request: invalid shard_id");
            for (int i = 0; i < merge_num; ++i) {
                int32_t shard_items_num;
                req >> shard_items_num;
                if (shard_items_num == 0) continue;
                std::vector<char> ar;
                ps_deserialize(req.lazy(), ar);
                PSHBM_SCHECK(ar.size() == (size_t)shard_items_num * st.record_bytes(), "block size mismatch");
                // The reference sets the items one after the other, so the last item of a key stays
                // (:548-560). pshbm_load wants distinct keys: keep the last record of each.
                const size_t rec = st.record_bytes();
                size_t kept = keep_last_of_each_key(ar.data(), (size_t)shard_items_num, rec);
                if (pshbm_load(st.get(shard_id), ar.data(), kept, 0) != PSHBM_OK) healthy = false;
            }
        }
        PSHBM_SCHECK(req.archive().is_exhausted(), "request not exhausted");
        if (healthy) {
            resp << Status();
        } else {
            resp.rpc_response().set_error_code(RpcErrorCodeType::ELOGICERROR);
            resp << Status::OOM("PServer OOM during direct push");
        }
    }
};

// ---- dense tables ----------------------------------------------------------------------------
// A dense parameter is a vector stored under a dense_key_t (an int64 id >= 0) and cut by the
// client's value partitioner into slices; the server keeps one map entry per slice under
// dense_slice_key_t {id, slice_id} (pico-ps/common/dense_common.h:19-104). On an HBM table a slice
// is one row of `dim` floats under the 64-bit key  id << 24 | slice_id  (ids below 2^39, slice ids
// below 2^24; the reference's empty and deleted slice keys have negative fields and cannot occur).
// Rows have one length, so every slice on the wire is exactly `dim` floats: the client uses
// HbmDenseValuePartitioner, which pads the last slice of a parameter with zeros, and
// HbmDenseValueMerger, which drops the padding again.
inline uint64_t dense_slice_key(int64_t id, int32_t slice_id) {
    PSHBM_SCHECK(id >= 0 && id < (int64_t(1) << 39) && slice_id >= 0 && slice_id < (1 << 24),
                 "dense slice key out of range");  // dense_common.h:77-83
    return (uint64_t)id << 24 | (uint32_t)slice_id;
}

// VAL_PARTITIONER of a dense table (the role of DenseValuePartitioner, dense_common.h:137-151, and of
// TestValuePartitioner, pico-ps/test/TestOps.h:307-319): slices of `block` elements, the last padded.
struct HbmDenseValuePartitioner {
    struct PartitionResult {
        std::vector<size_t> serialized_size;
        std::vector<std::vector<float>> parts;
    };
    explicit HbmDenseValuePartitioner(size_t block) : _block(block) {}
    PartitionResult partition(int64_t /*key*/, const std::vector<float>& origin) const {
        PartitionResult r;
        for (size_t l = 0; l < origin.size(); l += _block) {
            const size_t e = std::min(l + _block, origin.size());
            r.parts.emplace_back(origin.begin() + l, origin.begin() + e);
            r.parts.back().resize(_block, 0.0f);
            r.serialized_size.push_back(_block * sizeof(float));
        }
        return r;
    }

private:
    size_t _block;
};

// VAL_MERGER of a dense table (DenseValueMerger, dense_common.h:153-175; TestValueMerger,
// TestOps.h:321-335): slice `idx` lands at idx * block of the pulled vector, cut at its end.
struct HbmDenseValueMerger {
    explicit HbmDenseValueMerger(size_t block) : _block(block) {}
    size_t slice_number(int64_t /*key*/, const std::vector<float>& val) const { return (val.size() + _block - 1) / _block; }
    void merge(std::vector<float>& merged, const std::vector<float>& slice, size_t idx) const {
        const size_t at = idx * _block;
        PSHBM_SCHECK(at <= merged.size(), "dense slice beyond the pulled vector");
        std::copy(slice.begin(), slice.begin() + std::min(slice.size(), merged.size() - at), merged.begin() + at);
    }

private:
    size_t _block;
};

// Server halves of the dense push (DenseTablePushOperator, operator/DensePushOperator.h:137-316).
// Request: dense key, i32 shards_num; per shard {i32 shard_id, i32 shard_slices_num; per slice
// {i32 slice_id; one lazy block = the slice's push value, `dim` raw floats}} (:97-127). The slices
// of one shard go to the table as one batch. The update is the table's optimizer: a slice that is
// absent is created by its first push, as init_store_value of the test operator does
// (pico-ps/test/TestOps.h:355-359), a present one goes through store_push_value (:372-376).
class HbmDensePushOperator {
public:
    explicit HbmDensePushOperator(const Configure&) {}

    void apply_async_push_request(RuntimeInfo& rt, PSRequest& req, Storage* storage, Storage* /*incr_storage*/,
                                  PSResponse& resp) {  // :137-200
        Status status;
        for_each_shard(rt, req, storage, [&](pshbm_table* t, const std::vector<uint64_t>& keys, const std::vector<float>& vals) {
            int32_t rc = pshbm_push(t, keys.data(), vals.data(), keys.size(), 0);
            if (rc == PSHBM_OUT_OF_MEMORY) status = Status::OOM(pshbm_last_error(t));
            else if (rc != PSHBM_OK) status = Status::Error(pshbm_last_error(t));
        });
        PSHBM_SCHECK(req.archive().is_exhausted(), "request not exhausted");  // :197
        resp = PSResponse(req);
        if (!status.ok()) resp.rpc_response().set_error_code(RpcErrorCodeType::ELOGICERROR);
        resp << status;
    }

    // :202-253: the slices are merged into the delta storage (merge_push_value); here they are
    // queued in the shard's table and summed at the store.
    void apply_sync_push_request(RuntimeInfo& rt, PSRequest& req, Storage* storage, PSResponse& resp) {
        Status status;
        for_each_shard(rt, req, storage, [&](pshbm_table* t, const std::vector<uint64_t>& keys, const std::vector<float>& vals) {
            if (pshbm_queue(t, keys.data(), vals.data(), keys.size()) != PSHBM_OK) status = Status::Error(pshbm_last_error(t));
        });
        PSHBM_SCHECK(req.archive().is_exhausted(), "request not exhausted");  // :250
        resp = PSResponse(req);
        resp << status;
    }

    // :255-316: acknowledge first (:290-292), then apply every merged slice.
    void apply_store_request(RuntimeInfo& rt, PSRequest& req, Storage* delta_storage, Storage* storage,
                             Storage* /*incr_storage*/, std::function<void(PSResponse&&)> send_response) {
        int32_t shard_id;
        req >> shard_id;
        PSHBM_SCHECK(req.archive().is_exhausted(), "request not exhausted");                 // :262
        PSHBM_SCHECK(rt.local_shards().count(shard_id), "Bad Request: invalid shard_id");  // :263-264
        PSResponse resp(req);
        resp << Status();
        send_response(std::move(resp));
        if (delta_storage == nullptr) return;  // :266-271
        pshbm_store(static_cast<HbmShardStorage*>(storage)->get(shard_id), 0);
    }

    std::unique_ptr<Storage> create_delta_storage(RuntimeInfo&) { return std::make_unique<HbmDeltaStorage>(); }  // :325-327

private:
    template <class F>
    static void for_each_shard(RuntimeInfo& rt, PSRequest& req, Storage* storage, F&& f) {
        int64_t key;
        int32_t shards_num;
        req >> key >> shards_num;
        auto& st = *static_cast<HbmShardStorage*>(storage);
        const size_t dim = st.dim();
        std::vector<uint64_t> keys;
        std::vector<float> vals;
        while (shards_num--) {
            int32_t shard_id, shard_slices_num;
            req >> shard_id >> shard_slices_num;
            PSHBM_SCHECK(rt.local_shards().count(shard_id) != 0, "Bad Request: invalid shard_id");  // :157-158
            keys.clear();
            vals.clear();
            while (shard_slices_num--) {
                int32_t slice_id;
                req >> slice_id;
                std::vector<char> push_val;
                ps_deserialize(req.lazy(), push_val);
                PSHBM_SCHECK(push_val.size() == dim * 4, "dense slice is not `dim` floats");
                keys.push_back(dense_slice_key(key, slice_id));
                const float* v = reinterpret_cast<const float*>(push_val.data());
                vals.insert(vals.end(), v, v + dim);
            }
            if (!keys.empty()) f(st.get(shard_id), keys, vals);
        }
    }
};

// Server half of the dense pull (DenseTablePullOperator::apply_request, operator/DensePullOperator.h:118-181).
// Request: dense key, i32 shards_num; per shard {i32 shard_id, i32 shard_slices_num; the slice ids}
// (:100-112). Response: i32 shards_num; per shard {i32 shard_slices_num; per slice {i32 slice_id}},
// with one lazy block of `dim` floats per slice, in request order. A slice that is not stored is a
// programmer error there (SCHECK(it != ht.end()), :154) and here.
class HbmDensePullOperator {
public:
    explicit HbmDensePullOperator(const Configure&) {}
    void apply_request(RuntimeInfo& rt, PSRequest& req, Storage* storage, PSResponse& resp) {
        int64_t key;
        int32_t shards_num;
        req >> key >> shards_num;
        resp = PSResponse(req);
        resp << shards_num;
        bool healthy = true;
        std::string why;
        auto& st = *static_cast<HbmShardStorage*>(storage);
        const size_t dim = st.dim();
        std::vector<std::vector<char>> blocks;
        std::vector<uint64_t> keys;
        std::vector<float> rows;
        std::vector<uint8_t> hit;
        while (shards_num--) {
            int32_t shard_id, shard_slices_num;
            req >> shard_id >> shard_slices_num;
            resp << shard_slices_num;
            PSHBM_SCHECK(rt.local_shards().count(shard_id) != 0, "Bad Request: invalid shard_id");  // :140-141
            keys.clear();
            for (int32_t i = 0; i < shard_slices_num; ++i) {
                int32_t slice_id;
                req >> slice_id;
                resp << slice_id;
                keys.push_back(dense_slice_key(key, slice_id));
            }
            if (keys.empty()) continue;
            rows.resize(keys.size() * dim);
            hit.assign(keys.size(), 0);
            pshbm_table* t = st.get(shard_id);
            if (pshbm_pull(t, keys.data(), keys.size(), rows.data(), hit.data(), 0) != PSHBM_OK) {
                healthy = false;
                why = pshbm_last_error(t);
                continue;
            }
            for (size_t i = 0; i < keys.size(); ++i) {
                PSHBM_SCHECK(hit[i], "dense slice is not stored");  // :154
                const char* p = reinterpret_cast<const char*>(rows.data() + i * dim);
                blocks.emplace_back(p, p + dim * 4);
            }
        }
        PSHBM_SCHECK(req.archive().is_exhausted(), "request not exhausted");  // :180
        if (healthy) {
            for (auto& b : blocks) ps_serialize(resp.lazy(), std::move(b));
        } else {  // :170-179
            resp = PSResponse(req);
            resp.rpc_response().set_error_code(RpcErrorCodeType::ELOGICERROR);
            resp << Status::OOM("PServer OOM during dense pull: " + why);
        }
    }
};

// Result of the device for-each: what TestForEachResult {num, sum, count} generalises to
// (pico-ps/test/TestOps.h:152-157): the records visited and the sum of every value column.
struct HbmForEachResult {
    int64_t num = 0;
    std::vector<double> sums;
    void merge(const HbmForEachResult& in) {  // merge_result, TestOps.h:180-184
        num += in.num;
        if (sums.size() < in.sums.size()) sums.resize(in.sums.size(), 0.0);
        for (size_t i = 0; i < in.sums.size(); ++i) sums[i] += in.sums[i];
    }
    friend BinaryArchive& operator<<(BinaryArchive& ar, const HbmForEachResult& r) { return ar << r.num << r.sums; }
    friend BinaryArchive& operator>>(BinaryArchive& ar, HbmForEachResult& r) { return ar >> r.num >> r.sums; }
};

// Server half of the read-only for-each (SparseTableForEachReadOperator::apply_request,
// ForEachOperator.h:166-199). Request: i32 shard_id (a carried item would follow; this hook has
// none). Response: Status, then the result of that shard. The hook is the count / column-sum
// reduction over the records that satisfy `where` (none = all), evaluated on the device.
class HbmForEachOperator {
public:
    explicit HbmForEachOperator(const Configure&) { _where.struct_size = sizeof _where; }
    void set_where(const pshbm_predicate& w) { _where = w; }
    void apply_request(RuntimeInfo& rt, PSRequest& req, Storage* storage, PSResponse& resp_ret) {
        int32_t shard_id;
        req >> shard_id;
        PSHBM_SCHECK(req.archive().is_exhausted(), "Bad Request: trailing bytes");           // :176
        PSHBM_SCHECK(rt.local_shards().count(shard_id) != 0, "Bad Request: invalid shard_id");  // :177-178
        auto& st = *static_cast<HbmShardStorage*>(storage);
        HbmForEachResult res;
        res.sums.assign(st.value_floats(), 0.0);
        uint64_t count = 0;
        int32_t rc = pshbm_for_each(st.get(shard_id), _where.n_terms ? &_where : nullptr, &count, res.sums.data());
        PSHBM_SCHECK(rc == PSHBM_OK, std::string("for_each failed: ") + pshbm_last_error(st.get(shard_id)));
        res.num = (int64_t)count;
        PSResponse resp(req);
        resp << Status();
        resp.archive() << res;
        resp_ret = std::move(resp);
    }

private:
    pshbm_predicate _where{};
};

// Server half of erase-if (SparseTableEraseIfOperator::apply_request, EraseIfOperator.h:27-55).
// Request: i32 shard_id. Response: Status and an empty archive. The erase_if hook is `where`.
class HbmEraseIfOperator {
public:
    explicit HbmEraseIfOperator(const Configure&) { _where.struct_size = sizeof _where; }
    void set_where(const pshbm_predicate& w) { _where = w; }
    void apply_request(RuntimeInfo& rt, PSRequest& req, Storage* storage, PSResponse& resp_ret) {
        int32_t shard_id;
        req >> shard_id;
        PSHBM_SCHECK(req.archive().is_exhausted(), "Bad Request: trailing bytes");           // :34
        PSHBM_SCHECK(rt.local_shards().count(shard_id) != 0, "Bad Request: invalid shard_id");  // :35-36
        auto& st = *static_cast<HbmShardStorage*>(storage);
        int32_t rc = pshbm_erase_if(st.get(shard_id), _where.n_terms ? &_where : nullptr, nullptr);
        PSHBM_SCHECK(rc == PSHBM_OK, std::string("erase_if failed: ") + pshbm_last_error(st.get(shard_id)));
        PSResponse resp(req);
        BinaryArchive empty_ar;
        resp << Status();
        resp.archive() << empty_ar.size();
        resp_ret = std::move(resp);
    }

private:
    pshbm_predicate _where{};
};

struct DumpArgs {  // handler/DumpHandler.h: where to write and into how many files per node
    std::string uri;
    int32_t file_number = 1;
    friend BinaryArchive& operator<<(BinaryArchive& ar, const DumpArgs& a) { return ar << a.uri << a.file_number; }
    friend BinaryArchive& operator>>(BinaryArchive& ar, DumpArgs& a) { return ar >> a.uri >> a.file_number; }
};

// BaseKVTextFileDumpOperator::apply_request, DumpOperator.h:137-183. Request: DumpArgs, i32 file_id,
// vector of shard ids (:66-80). DS_WRITER: bool open(const std::string&), bool write(uint64_t key,
// const float* value, uint32_t value_floats), void close() -- the record encoding stays with the host.
template <class DS_WRITER>
class HbmDumpOperator {
public:
    explicit HbmDumpOperator(const Configure& config) : _block((size_t)config.number("block_size", 65536)) {}
    void apply_request(RuntimeInfo& rt, PSRequest& req, Storage* storage, PSResponse& resp_ret) {
        DumpArgs args;
        int32_t file_id;
        std::vector<int32_t> shard_ids;
        req.archive() >> args >> file_id >> shard_ids;
        PSHBM_SCHECK(req.archive().is_exhausted(), "request not exhausted");
        DS_WRITER writer;
        const std::string name = args.uri + "/model_" + std::to_string(rt.node_id()) + "_" + std::to_string(file_id);  // :156
        PSHBM_SCHECK(writer.open(name), "failed to open file for write: " + name);
        auto& st = *static_cast<HbmShardStorage*>(storage);
        const size_t rec = st.record_bytes();
        for (int32_t shard_id : shard_ids) {
            for (size_t off = 0;;) {  // the shard streams out in slab order, block by block
                BinaryArchive ar;
                size_t got = st.iterate_batch_as_binary_archive(shard_id, off, _block, ar);
                for (size_t i = 0; i < got; ++i) {
                    uint64_t key;
                    std::memcpy(&key, ar.buffer().data() + i * rec, 8);
                    PSHBM_SCHECK(writer.write(key, reinterpret_cast<const float*>(ar.buffer().data() + i * rec + 8),
                                              st.value_floats()),
                                 "failed to write");
                }
                off += got;
                if (got < _block) break;
            }
        }
        writer.close();
        PSResponse resp(req);
        resp << Status();
        resp_ret = std::move(resp);
    }

private:
    size_t _block;
};

// BaseKVTextFileLoadOperator::restore, LoadOperator.h:164-213: every record of the files whose key
// belongs to a local shard is inserted, block_size records at a time; a key that is already there
// aborts (SCHECK(insert.second), :194,210). DS_READER: bool open(const std::string&),
// bool read(uint64_t& key, float* value). `partition` maps a key to its shard id (one shard: 0).
template <class DS_READER>
class HbmLoadOperator {
public:
    explicit HbmLoadOperator(const Configure& config) : _block_size((size_t)config.number("block_size", 1000)) {}
    void restore(const std::vector<std::string>& files, RuntimeInfo& rt, Storage* storage,
                 const std::function<int32_t(uint64_t)>& partition) {
        auto& st = *static_cast<HbmShardStorage*>(storage);
        const size_t rec = st.record_bytes();
        std::map<int32_t, std::vector<char>> pending;
        auto flush = [&](int32_t shard_id, std::vector<char>& buf) {
            if (buf.empty()) return;
            int32_t rc = pshbm_load(st.get(shard_id), buf.data(), buf.size() / rec, PSHBM_LOAD_UNIQUE);
            PSHBM_SCHECK(rc == PSHBM_OK, std::string("restore: ") + pshbm_last_error(st.get(shard_id)));
            buf.clear();
        };
        std::vector<char> one(rec);
        for (const std::string& f : files) {
            DS_READER reader;
            PSHBM_SCHECK(reader.open(f), "failed to open " + f);
            uint64_t key;
            while (reader.read(key, reinterpret_cast<float*>(one.data() + 8))) {
                const int32_t shard_id = partition(key);
                if (rt.local_shards().count(shard_id) == 0) continue;  // :185-186
                std::memcpy(one.data(), &key, 8);
                auto& buf = pending[shard_id];
                buf.insert(buf.end(), one.begin(), one.end());
                if (buf.size() >= _block_size * rec) flush(shard_id, buf);
            }
        }
        for (auto& p : pending) flush(p.first, p.second);
    }

private:
    size_t _block_size;
};

// The key partitioner of sparse tables: DefaultPartitioner<uint64_t> (common/Partitioner.h:43-61),
// partition = jump_consistent_hash(murmur_hash(key), n). pico-core's two functions are not in the
// reference tree; these are the published ones (MurmurHash3's 64-bit finalizer, Lamping and Veach's
// jump consistent hash), which the library also evaluates on the device: a partitioner that
// declares `device_terms` lets HbmShuffleOperator purge a shard with one erase_if on the device
// instead of walking its keys over the link.
struct HbmDefaultPartitioner {
    static constexpr bool device_terms = true;
    int32_t partition(uint64_t key, int32_t num_buckets) const { return pshbm_partition(key, num_buckets); }
};
template <class P, class = void>
struct hbm_partitioner_on_device : std::false_type {};
template <class P>
struct hbm_partitioner_on_device<P, std::enable_if_t<P::device_terms>> : std::true_type {};

// Re-sharding after the set of servers changed (UpdateContextOperator.h:100-305). The host logic
// that drives it stays as it is; what it needs from the storage is (1) the items of a shard that
// now belong elsewhere, a bounded block at a time, and (2) the purge of those items.
// PARTITIONER::partition(key, global_shard_num) is the reference's key partitioner
// (common/Partitioner.h:43-61), evaluated on the host -- except in the purge, which runs on the
// device when the partitioner is the library's (HbmDefaultPartitioner).
template <class PARTITIONER>
class HbmShuffleOperator {
public:
    explicit HbmShuffleOperator(const Configure& config)
        : _block_items((size_t)config.number("shuffle_block_items", 4096)) {}

    // PushItemsGenerator (UpdateContextOperator.h:214-297): walks the shard in slab order and hands
    // out the items whose partition is no longer `shard_id` (all items when the shard changes node).
    class PushItemsGenerator {
    public:
        PushItemsGenerator(HbmShardStorage& st, int32_t shard_id, int32_t global_shard_num, bool shard_node_change,
                           size_t block_items, PARTITIONER& partitioner)
            : _st(st), _shard_id(shard_id), _global_shard_num(global_shard_num),
              _shard_node_change(shard_node_change), _block_items(block_items), _partitioner(partitioner) {}
        // Appends up to one block of (key, value) to keys / vals; returns how many. 0 = finished.
        size_t generate_push_items(std::vector<uint64_t>& keys, std::vector<float>& vals) {
            const size_t rec = _st.record_bytes(), vf = _st.value_floats();
            std::vector<char> buf(_block_items * rec);
            size_t count = 0;
            while (count == 0 && !_finished) {
                size_t got = 0;
                int32_t rc = pshbm_iterate(_st.get(_shard_id), _offset, _block_items, buf.data(), &got);
                PSHBM_SCHECK(rc == PSHBM_OK, "iterate failed");
                _offset += got;
                _finished = got < _block_items;
                for (size_t i = 0; i < got; ++i) {
                    uint64_t key;
                    std::memcpy(&key, buf.data() + i * rec, 8);
                    if (_partitioner.partition(key, _global_shard_num) != _shard_id || _shard_node_change) {  // :273-277
                        keys.push_back(key);
                        const float* v = reinterpret_cast<const float*>(buf.data() + i * rec + 8);
                        vals.insert(vals.end(), v, v + vf);
                        ++count;
                    }
                }
            }
            return count;
        }

    private:
        HbmShardStorage& _st;
        int32_t _shard_id, _global_shard_num;
        bool _shard_node_change;
        size_t _block_items, _offset = 0;
        bool _finished = false;
        PARTITIONER& _partitioner;
    };

    std::unique_ptr<PushItemsGenerator> lock_push_items_generator(RuntimeInfo& new_rt, Storage* storage,
                                                                  int32_t shard_id, bool shard_node_change) {
        return std::make_unique<PushItemsGenerator>(*static_cast<HbmShardStorage*>(storage), shard_id,
                                                    new_rt.global_shard_num(), shard_node_change, _block_items,
                                                    _key_partitioner);
    }

    // apply_purge_request (UpdateContextOperator.h:143-196): a shard that stays local keeps only the
    // keys that still map to it, and its hash array is rebuilt (safe_shrink); any other shard goes.
    void apply_purge_request(RuntimeInfo& new_rt, PSRequest& req, Storage* storage, PSResponse& resp) {
        auto& st = *static_cast<HbmShardStorage*>(storage);
        int32_t shard_id;
        req >> shard_id;
        if (new_rt.local_shards().count(shard_id)) {
            pshbm_table* t = st.get(shard_id);
            if constexpr (hbm_partitioner_on_device<PARTITIONER>::value) {
                pshbm_predicate not_mine{};
                not_mine.struct_size = sizeof not_mine;
                not_mine.n_terms = 1;
                not_mine.term[0].column = PSHBM_COL_KEY;
                not_mine.term[0].cmp = PSHBM_CMP_PART_NE;
                not_mine.term[0].u = (uint64_t)new_rt.global_shard_num();
                not_mine.term[0].u2 = (uint64_t)shard_id;
                PSHBM_SCHECK(pshbm_erase_if(t, &not_mine, nullptr) == PSHBM_OK, "erase_if failed");
            } else {
                std::vector<uint64_t> keys(_block_items), gone;
                for (size_t offset = 0;;) {  // the keys first: erasing moves rows, which would disturb the walk
                    size_t got = 0;
                    PSHBM_SCHECK(pshbm_iterate_keys(t, offset, _block_items, keys.data(), &got) == PSHBM_OK, "iterate failed");
                    for (size_t i = 0; i < got; ++i)
                        if (_key_partitioner.partition(keys[i], new_rt.global_shard_num()) != shard_id) gone.push_back(keys[i]);
                    offset += got;
                    if (got < _block_items) break;
                }
                PSHBM_SCHECK(pshbm_erase(t, gone.data(), gone.size(), nullptr) == PSHBM_OK, "erase failed");
            }
            PSHBM_SCHECK(pshbm_compact(t) == PSHBM_OK, "compact failed");
        } else {
            st.erase_shard(shard_id);
        }
        resp = PSResponse(req);
        resp << Status();
    }

private:
    size_t _block_items;
    PARTITIONER _key_partitioner;
};

// Sync to another cluster (KVSyncOperator, operator/SyncOperator.h:102-266): the values that pushes
// wrote since the last sync travel to the storage of, say, an online-serving cluster. The sending
// side walks the increment -- here the marks inside each shard's table, taken once per walk
// (IncrementStorage::read_storage, service/IncrementStorage.h:29-36) -- and cuts it into requests
// of up to block_size items, partitioned for the receiving cluster's shards; the receiving side
// upserts them (ht[key] = value, :159-163). to_sync_value (:186) is the identity: the whole value
// travels. PARTITIONER::partition(key, global_shard_num) as in HbmShuffleOperator.
template <class PARTITIONER>
class HbmSyncOperator {
public:
    explicit HbmSyncOperator(const Configure& config) : _block_size((size_t)config.number("block_size", 1000)) {}  // :24

    // TemplateStorageIterator over the increment (:45-98): the records {key, value} every local
    // shard's pushes touched, in the order the shards and their slabs give.
    class IncrIterator {
    public:
        IncrIterator(HbmShardStorage& st) : _rec(st.record_bytes()) {
            for (int32_t shard_id : st.shard_list()) {
                uint64_t marked = 0;
                PSHBM_SCHECK(pshbm_increment_size(st.get(shard_id), &marked) == PSHBM_OK, "increment_size failed");
                if (marked == 0) continue;
                const size_t at = _records.size();
                _records.resize(at + marked * _rec);
                size_t got = 0;
                PSHBM_SCHECK(pshbm_take_increment(st.get(shard_id), _records.data() + at, marked, &got) == PSHBM_OK,
                             "take_increment failed");
                _records.resize(at + got * _rec);
            }
        }
        const char* next() {  // nullptr at the end
            if (_pos >= _records.size()) return nullptr;
            const char* p = _records.data() + _pos;
            _pos += _rec;
            return p;
        }
        size_t record_bytes() const { return _rec; }

    private:
        std::vector<char> _records;
        size_t _rec, _pos = 0;
    };

    std::unique_ptr<IncrIterator> incr_iterator(Storage* storage) {  // :188-190
        return std::make_unique<IncrIterator>(*static_cast<HbmShardStorage*>(storage));
    }

    // generate_sync_request, :192-214 + generate_request, :217-258: one request per node of the
    // receiving cluster `rt`: i32 node_items, i32 n_shards, then per shard i32 shard_id,
    // i32 shard_items and the items as {key, value} records. Status::Empty when nothing is left.
    Status generate_sync_request(IncrIterator* it, RuntimeInfo& rt, std::vector<PSRequest>& reqs) {
        std::vector<std::vector<char>> tables(rt.global_shard_num());
        const size_t rec = it->record_bytes();
        size_t cnt = 0;
        for (; cnt < _block_size; ++cnt) {
            const char* item = it->next();
            if (item == nullptr) break;
            uint64_t key;
            std::memcpy(&key, item, 8);
            std::vector<char>& tb = tables[_key_partitioner.partition(key, rt.global_shard_num())];
            tb.insert(tb.end(), item, item + rec);
        }
        if (cnt == 0) return Status::Empty("");
        for (auto& node : rt.nodes()) {
            if (node.second.empty()) return Status::NoReplica("");
            int32_t node_items = 0;
            for (int32_t shard_id : node.second) node_items += (int32_t)(tables[shard_id].size() / rec);
            reqs.emplace_back();
            BinaryArchive& ar = reqs.back().archive();
            ar << node_items << (int32_t)node.second.size();
            for (int32_t shard_id : node.second) {
                ar << shard_id << (int32_t)(tables[shard_id].size() / rec);
                ar.write_raw(tables[shard_id].data(), tables[shard_id].size());
            }
        }
        return Status();
    }

    // apply_sync_request, :126-184. The items of a shard lie in the archive as the records
    // pshbm_load takes; a shard that cannot hold them grows like one that a push fills, and past
    // its limit the response carries Status::OOM (:164-168).
    void apply_sync_request(RuntimeInfo& rt, PSRequest& req, Storage* storage, PSResponse& resp_ret) {
        BinaryArchive& ar = req.archive();
        auto& st = *static_cast<HbmShardStorage*>(storage);
        const size_t rec = st.record_bytes();
        int32_t node_items, n_shards;
        ar >> node_items >> n_shards;
        Status status;
        while (n_shards--) {
            int32_t shard_id, shard_items;
            ar >> shard_id;
            PSHBM_SCHECK(rt.local_shards().count(shard_id) != 0, "Bad Request: invalid shard_id");
            ar >> shard_items;
            node_items -= shard_items;
            PSHBM_SCHECK(ar.readable() >= (size_t)shard_items * rec, "sync block size mismatch");
            if (status.ok() && shard_items > 0) {
                pshbm_table* t = st.get(shard_id);
                auto lk = st.lock_shard(shard_id);
                int32_t rc = pshbm_load(t, ar.cursor(), (size_t)shard_items, 0);
                while (rc == PSHBM_OUT_OF_MEMORY && st.grow(shard_id)) rc = pshbm_load(t, ar.cursor(), (size_t)shard_items, 0);
                if (rc == PSHBM_OUT_OF_MEMORY) status = Status::OOM("PServer OOM during sync op");
                else if (rc != PSHBM_OK) status = Status::Error(pshbm_last_error(t));
            }
            ar.advance((size_t)shard_items * rec);
        }
        PSHBM_SCHECK(node_items == 0, "sync request: item counts do not add up");  // :178
        PSHBM_SCHECK(ar.is_exhausted(), "request not exhausted");                  // :179
        resp_ret = PSResponse(req);
        resp_ret << status;
    }

private:
    size_t _block_size;
    PARTITIONER _key_partitioner;
};

// Coordinated restore of a dead node's shard from a live replica (RestoreOperator.h:100-151): the
// serving side answers (offset, batch) slices of a shard, the restoring side inserts what it gets
// and keeps what it already has.
class HbmRestoreOperator {
public:
    explicit HbmRestoreOperator(const Configure&) {}
    void apply_coordinated_restore_request(PSRequest& req, Storage* storage, PSResponse& resp) {
        int32_t storage_id, iterator_id, shard_id;
        uint64_t offset, batch_size;
        req >> storage_id >> iterator_id >> offset >> batch_size >> shard_id;
        auto& st = *static_cast<HbmShardStorage*>(storage);
        if (st.get(shard_id) == nullptr) {  // :111-115
            resp.rpc_response().set_error_code(RpcErrorCodeType::ELOGICERROR);
            resp << Status::InvalidID("Invalid shard id");
            return;
        }
        BinaryArchive ar;
        const size_t num = st.iterate_batch_as_binary_archive(shard_id, offset, batch_size, ar);
        const bool finished = num < batch_size;
        resp = PSResponse(req);
        resp << storage_id << shard_id << finished << iterator_id << (uint64_t)(offset + num) << (uint64_t)num;
        ps_serialize(resp.lazy(), std::move(ar.buffer()));
    }
    // returns {finished, next_offset}
    std::pair<bool, uint64_t> apply_coordinated_restore_response(PSResponse& resp, Storage* storage) {
        int32_t storage_id, shard_id, iterator_id;
        bool finished;
        uint64_t next_offset, num;
        resp >> storage_id >> shard_id >> finished >> iterator_id >> next_offset >> num;
        std::vector<char> block;
        ps_deserialize(resp.lazy(), block);
        auto& st = *static_cast<HbmShardStorage*>(storage);
        const size_t rec = st.record_bytes();
        PSHBM_SCHECK(block.size() == num * rec, "restore block size mismatch");
        // ht.insert keeps a key that is present (:141-146): drop those records before the load
        std::vector<uint64_t> keys(num);
        for (size_t i = 0; i < num; ++i) std::memcpy(&keys[i], block.data() + i * rec, 8);
        std::vector<float> rows(num * st.dim());
        std::vector<uint8_t> hit(num);
        pshbm_table* t = st.get(shard_id);
        PSHBM_SCHECK(pshbm_pull(t, keys.data(), num, rows.data(), hit.data(), 0) == PSHBM_OK, "pull failed");
        std::vector<char> fresh;
        for (size_t i = 0; i < num; ++i)
            if (!hit[i]) fresh.insert(fresh.end(), block.begin() + i * rec, block.begin() + (i + 1) * rec);
        PSHBM_SCHECK(pshbm_load(t, fresh.data(), fresh.size() / rec, PSHBM_LOAD_UNIQUE) == PSHBM_OK, "load failed");
        return {finished, next_offset};
    }
};

}  // namespace pshbm_host
