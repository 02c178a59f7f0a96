// Drives the host-side operator mirror (parameter-server_amd/host/hbm_ops.h) the way the
// reference's test_sparse drives its operators (pico-ps/test/ps_service_test.cpp:77-184), but in
// one process and through hand-built wire requests: every "rank" pushes keys
// [rank*100, (rank+1)*100) with arg = key once asynchronously and once (even ranks twice)
// synchronously, the store is applied, the table is dumped to files, restored into a new storage,
// and pulled. The test operator of the reference (TestValue{sum,count}, TestOps.h:53-118) is the
// dim-2 SUM table: a push of arg = key is the gradient [key, 1].
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include <thread>

#include "../../parameter-server_amd/host/hbm_ops.h"

using namespace pshbm_host;

static int g_failed = 0;
#define EXPECT(cond)                                                              \
    do {                                                                          \
        if (!(cond)) {                                                            \
            std::printf("EXPECT failed at line %d: %s\n", __LINE__, #cond);       \
            ++g_failed;                                                           \
        }                                                                         \
    } while (0)

constexpr int TEST_KEY_NUM = 100;  // pico-ps/test/TestOps.h:12
constexpr int NUM_RANKS = 3;
constexpr int NUM_SHARDS = 2;
static int32_t partition(uint64_t key) { return (int32_t)(key % NUM_SHARDS); }

struct Pair {  // std::pair<KEY, PUSH_VALUE> of the wire, SparsePushOperator.h:176-177
    uint64_t key;
    float v[2];
};
static_assert(sizeof(Pair) == 16, "wire pair is packed");

// Client half of a push for one client batch (generate_push_request, SparsePushOperator.h:156-185).
static PSRequest make_push_request(const std::vector<uint64_t>& keys, const std::vector<float>& args) {
    std::vector<std::vector<Pair>> by_shard(NUM_SHARDS);
    for (size_t i = 0; i < keys.size(); ++i) by_shard[partition(keys[i])].push_back({keys[i], {args[i], 1.0f}});
    PSRequest req;
    req << (int32_t)NUM_SHARDS << (int32_t)1;
    for (int32_t s = 0; s < NUM_SHARDS; ++s) {
        req << s << (int32_t)by_shard[s].size();
        if (!by_shard[s].empty()) {
            const char* p = reinterpret_cast<const char*>(by_shard[s].data());
            req.lazy().emplace_back(p, p + by_shard[s].size() * sizeof(Pair));
        }
    }
    return req;
}

// Client half of a pull (generate_request, SparsePullOperator.h:112-154) and of its response
// (apply_response + fill_pull_items, :256-304), for one unmerged request.
static std::vector<float> pull(HbmSparsePullOperator& op, RuntimeInfo& rt, Storage* st,
                               const std::vector<uint64_t>& keys, bool* ok) {
    std::vector<std::vector<uint64_t>> by_shard(NUM_SHARDS);
    std::vector<std::vector<size_t>> where(NUM_SHARDS);
    for (size_t i = 0; i < keys.size(); ++i) {
        by_shard[partition(keys[i])].push_back(keys[i]);
        where[partition(keys[i])].push_back(i);
    }
    PSRequest req;
    req << (int32_t)NUM_SHARDS << (int32_t)1;
    for (int32_t s = 0; s < NUM_SHARDS; ++s) {
        req << s << (int32_t)by_shard[s].size();
        if (!by_shard[s].empty()) {
            const char* p = reinterpret_cast<const char*>(by_shard[s].data());
            req.lazy().emplace_back(p, p + by_shard[s].size() * 8);
        }
    }
    PSResponse resp;
    op.apply_request(rt, req, st, resp);
    std::vector<float> out(keys.size() * 2, -3.0f);
    *ok = resp.error_code() == RpcErrorCodeType::SUCC;
    if (!*ok) return out;
    int32_t shards_num;
    resp >> shards_num;
    std::vector<int32_t> ids(shards_num);
    for (auto& id : ids) resp >> id;
    std::vector<char> values;
    ps_deserialize(resp.lazy(), values);
    const float* v = reinterpret_cast<const float*>(values.data());
    size_t at = 0;
    for (int32_t id : ids)
        for (size_t i : where[id]) {
            out[i * 2] = v[at * 2];
            out[i * 2 + 1] = v[at * 2 + 1];
            ++at;
        }
    EXPECT(at * 8 == values.size());
    return out;
}

struct FileWriter {  // stands for TestDsWriter (pico-ps/test/TestOpsDs.h:13-45)
    std::ofstream f;
    bool open(const std::string& name) {
        f.open(name, std::ios::binary);
        return f.good();
    }
    bool write(uint64_t key, const float* value, uint32_t vf) {
        f.write(reinterpret_cast<const char*>(&key), 8);
        f.write(reinterpret_cast<const char*>(value), vf * 4);
        return f.good();
    }
    void close() { f.close(); }
};
struct FileReader {  // stands for TestDsReader (TestOpsDs.h:47-75); dim-2 SUM values
    std::ifstream f;
    bool open(const std::string& name) {
        f.open(name, std::ios::binary);
        return f.good();
    }
    bool read(uint64_t& key, float* value) {
        f.read(reinterpret_cast<char*>(&key), 8);
        f.read(reinterpret_cast<char*>(value), 8);
        return f.good();
    }
};


// ---- dense tables: the flow of test_dense (pico-ps/test/ps_service_test.cpp:241-409) -------------
// Every "rank" owns the dense keys [rank*100, (rank+1)*100); the parameter of key k is the vector
// {k, k+1, ..., 2k-1} (k elements, :262-266), cut into slices of DENSE_BLOCK_SIZE = 5
// (pico-ps/test/TestOps.h:270); the test operator adds what is pushed (TestOps.h:351-377).
static constexpr size_t DENSE_BLOCK_SIZE = 5;
static int32_t dense_partition(int64_t key, int32_t slice_id) { return (int32_t)((key * 31 + slice_id) % NUM_SHARDS); }

static std::vector<float> dense_arg(int32_t key) {
    std::vector<float> v(key);
    for (int32_t i = 0; i < key; ++i) v[i] = (float)(key + i);
    return v;
}

// generate_push_request of the dense push (operator/DensePushOperator.h:89-131)
static bool make_dense_push_request(int64_t key, const std::vector<float>& arg, PSRequest& req) {
    HbmDenseValuePartitioner partitioner(DENSE_BLOCK_SIZE);
    auto parted = partitioner.partition(key, arg);
    std::vector<std::vector<int32_t>> shards_slices(NUM_SHARDS);
    for (size_t slice_id = 0; slice_id < parted.parts.size(); ++slice_id)
        shards_slices[dense_partition(key, (int32_t)slice_id)].push_back((int32_t)slice_id);
    req << key << (int32_t)NUM_SHARDS;
    int32_t total = 0;
    for (int32_t shard_id = 0; shard_id < NUM_SHARDS; ++shard_id) {
        req << shard_id << (int32_t)shards_slices[shard_id].size();
        for (int32_t slice_id : shards_slices[shard_id]) {
            req << slice_id;
            const auto& part = parted.parts[slice_id];
            const char* p = reinterpret_cast<const char*>(part.data());
            ps_serialize(req.lazy(), std::vector<char>(p, p + part.size() * 4));
            ++total;
        }
    }
    return total != 0;  // a request without slices is not sent (:127-129)
}

// generate_request + apply_response of the dense pull (operator/DensePullOperator.h:60-116, 183-221)
static std::vector<float> dense_pull(HbmDensePullOperator& op, RuntimeInfo& rt, Storage* st, int64_t key, size_t len) {
    HbmDenseValueMerger merger(DENSE_BLOCK_SIZE);
    std::vector<float> pull_arg(len, -1.0f);
    const int32_t slices_num = (int32_t)merger.slice_number(key, pull_arg);
    if (slices_num == 0) return pull_arg;
    std::vector<std::vector<int32_t>> shards_slices(NUM_SHARDS);
    for (int32_t slice_id = 0; slice_id < slices_num; ++slice_id) shards_slices[dense_partition(key, slice_id)].push_back(slice_id);
    PSRequest req;
    req << key << (int32_t)NUM_SHARDS;
    for (int32_t shard_id = 0; shard_id < NUM_SHARDS; ++shard_id) {
        req << shard_id << (int32_t)shards_slices[shard_id].size();
        for (int32_t slice_id : shards_slices[shard_id]) req << slice_id;
    }
    PSResponse resp;
    op.apply_request(rt, req, st, resp);
    EXPECT(resp.error_code() == RpcErrorCodeType::SUCC);
    int32_t shards_num;
    resp >> shards_num;
    int32_t seen = 0;
    while (shards_num--) {
        int32_t shard_slices_num;
        resp >> shard_slices_num;
        while (shard_slices_num--) {
            int32_t slice_id;
            resp >> slice_id;
            EXPECT(0 <= slice_id && slice_id < slices_num);
            std::vector<char> block;
            ps_deserialize(resp.lazy(), block);
            EXPECT(block.size() == DENSE_BLOCK_SIZE * 4);
            std::vector<float> slice(DENSE_BLOCK_SIZE);
            std::memcpy(slice.data(), block.data(), block.size());
            merger.merge(pull_arg, slice, slice_id);
            ++seen;
        }
    }
    EXPECT(seen == slices_num && resp.archive().is_exhausted() && resp.lazy().empty());
    return pull_arg;
}

template <size_t VF>
struct FixedReader {
    std::ifstream f;
    bool open(const std::string& name) {
        f.open(name, std::ios::binary);
        return f.good();
    }
    bool read(uint64_t& key, float* value) {
        f.read(reinterpret_cast<char*>(&key), 8);
        f.read(reinterpret_cast<char*>(value), VF * 4);
        return f.good();
    }
};

static void test_dense(const std::string& dir) {
    Configure op_config;
    op_config.set("dim", (double)DENSE_BLOCK_SIZE);
    op_config.set("optimizer", "sum");
    op_config.set("hbm_table.expected_max_items", 40000);
    op_config.set("block_size", 100);
    RuntimeInfo rt(0, {0, 1});
    HbmStorageOperator storage_op(op_config);
    std::unique_ptr<Storage> storage = storage_op.create_storage(rt, 0);
    HbmDensePushOperator push_op(op_config);
    HbmDensePullOperator pull_op(op_config);
    std::unique_ptr<Storage> delta = push_op.create_delta_storage(rt);
    const int32_t max_key = NUM_RANKS * TEST_KEY_NUM;

    auto push = [&](int32_t key, bool sync) {
        PSRequest req;
        if (!make_dense_push_request(key, dense_arg(key), req)) return;
        PSResponse resp;
        Status status;
        if (sync) push_op.apply_sync_push_request(rt, req, storage.get(), resp);
        else push_op.apply_async_push_request(rt, req, storage.get(), nullptr, resp);
        resp >> status;
        EXPECT(status.ok());
    };
    auto store = [&]() {
        for (int32_t shard = 0; shard < NUM_SHARDS; ++shard) {
            PSRequest req;
            req << shard;
            bool acked = false;
            push_op.apply_store_request(rt, req, delta.get(), storage.get(), nullptr, [&](PSResponse&& r) {
                Status s;
                r >> s;
                acked = s.ok();
            });
            EXPECT(acked);
        }
    };
    auto expect_all = [&](HbmDensePullOperator& op, Storage* st, int odd_factor, int even_factor) {
        for (int32_t key = 0; key < max_key; ++key) {
            const int rank = key / TEST_KEY_NUM;
            const float f = (float)(rank % 2 == 0 ? even_factor : odd_factor);
            auto got = dense_pull(op, rt, st, key, key);
            bool same = got.size() == (size_t)key;
            for (int32_t i = 0; same && i < key; ++i) same = got[i] == (float)(key + i) * f;
            EXPECT(same);
        }
    };
    for (int32_t key = 0; key < max_key; ++key) {  // :259-272
        push(key, false);
        push(key, true);
    }
    store();                                         // :274-277
    for (int32_t key = 0; key < max_key; ++key)      // :280-291: even ranks once more
        if ((key / TEST_KEY_NUM) % 2 == 0) push(key, true);
    store();                                         // :296-298
    expect_all(pull_op, storage.get(), 2, 3);
    for (int32_t key = 0; key < max_key; ++key) {    // :307-326
        push(key, false);
        push(key, true);
        if ((key / TEST_KEY_NUM) % 2 == 0) push(key, true);
    }
    expect_all(pull_op, storage.get(), 3, 4);        // :332-347: (key + i) * (3 + (rank even)); the queue is not applied yet
    store();                                         // :356-357
    // one table row per slice of DENSE_BLOCK_SIZE elements
    uint64_t slices = 0;
    for (int32_t key = 0; key < max_key; ++key) slices += (key + DENSE_BLOCK_SIZE - 1) / DENSE_BLOCK_SIZE;
    auto* hst = static_cast<HbmShardStorage*>(storage.get());
    EXPECT(hst->shard_size(0) + hst->shard_size(1) == slices);

    // dump (:359-361), then load into a storage created anew (:368-377) and pull (:393-409)
    HbmDumpOperator<FileWriter> dump_op(op_config);
    std::vector<std::string> files;
    for (int32_t file_id = 0; file_id < 2; ++file_id) {
        PSRequest req;
        DumpArgs args{dir, 2};
        std::vector<int32_t> shard_ids{file_id};
        req.archive() << args << file_id << shard_ids;
        PSResponse resp;
        dump_op.apply_request(rt, req, storage.get(), resp);
        Status status;
        resp >> status;
        EXPECT(status.ok());
        files.push_back(dir + "/model_0_" + std::to_string(file_id));
    }
    std::unique_ptr<Storage> loaded = storage_op.create_storage(rt, 1);
    HbmLoadOperator<FixedReader<DENSE_BLOCK_SIZE>> load_op(op_config);
    load_op.restore(files, rt, loaded.get(), [](uint64_t k) { return dense_partition((int64_t)(k >> 24), (int32_t)(k & 0xFFFFFF)); });
    HbmDensePullOperator pull_loaded(op_config);
    expect_all(pull_loaded, loaded.get(), 4, 6);     // (key + i) * (2 + (rank even)) * 2, :401

    // a slice that was never pushed is a programmer error (DensePullOperator.h:154)
    bool threw = false;
    try {
        dense_pull(pull_loaded, rt, loaded.get(), max_key + 7, 12);
    } catch (const std::logic_error&) {
        threw = true;
    }
    EXPECT(threw);
    // a slice of the wrong length is refused
    threw = false;
    try {
        PSRequest req;
        req << (int64_t)3 << (int32_t)1 << (int32_t)0 << (int32_t)1 << (int32_t)0;
        ps_serialize(req.lazy(), std::vector<char>(12));
        PSResponse resp;
        push_op.apply_async_push_request(rt, req, storage.get(), nullptr, resp);
    } catch (const std::logic_error&) {
        threw = true;
    }
    EXPECT(threw);
}

// A storage created for 64 keys takes 1000: the push that finds the table full grows it (twice the
// capacity at a time, up to hbm_table.grow_limit) and is applied again; past the limit the response
// carries Status::OOM, as the reference's does once its memory limit is reached
// (pico-ps/operator/SparsePullOperator.h:245-253).
static void test_growth() {
    Configure op_config;
    op_config.set("dim", 2);
    op_config.set("optimizer", "sum");
    op_config.set("hbm_table.expected_max_items", 64);
    op_config.set("hbm_table.grow_limit", 700);
    RuntimeInfo rt(0, {0, 1});
    HbmStorageOperator storage_op(op_config);
    std::unique_ptr<Storage> storage = storage_op.create_storage(rt, 0);
    HbmSparsePushOperator push_op(op_config);
    HbmSparsePullOperator pull_op(op_config);
    std::vector<uint64_t> keys;
    std::vector<float> args;
    for (int k = 0; k < 1000; ++k) {
        keys.push_back(k);
        args.push_back((float)k);
    }
    PSResponse resp;
    Status status;
    PSRequest a = make_push_request(keys, args);  // 500 keys per shard: 64 -> 128 -> 256 -> 512
    push_op.apply_async_push_request(rt, a, storage.get(), nullptr, resp);
    resp >> status;
    EXPECT(status.ok());
    auto* hst = static_cast<HbmShardStorage*>(storage.get());
    EXPECT(hst->shard_size(0) == 500 && hst->shard_size(1) == 500);
    bool ok;
    auto v = pull(pull_op, rt, storage.get(), keys, &ok);
    EXPECT(ok);
    for (size_t i = 0; i < keys.size(); ++i) EXPECT(v[i * 2] == (float)keys[i] && v[i * 2 + 1] == 1.0f);
    // 800 more keys: 400 per shard do not fit under the limit of 700
    std::vector<uint64_t> more;
    std::vector<float> margs;
    for (int k = 1000; k < 1800; ++k) {
        more.push_back(k);
        margs.push_back(1.0f);
    }
    PSRequest b = make_push_request(more, margs);
    PSResponse resp2;
    push_op.apply_async_push_request(rt, b, storage.get(), nullptr, resp2);
    Status status2;
    resp2 >> status2;
    EXPECT(status2.IsOOM() && resp2.error_code() == RpcErrorCodeType::ELOGICERROR);
    EXPECT(hst->shard_size(0) == 500 && hst->shard_size(1) == 500);
}

// A device memory limit (the hard limit of ShardStorageMemory, storage/Storage.cpp:93-98): growth
// that would pass it answers Status::OOM and leaves the shard as it was; with the limit lifted the
// same request goes through.
static void test_memory_limit() {
    Configure op_config;
    op_config.set("dim", 64);
    op_config.set("optimizer", "sum");
    op_config.set("hbm_table.expected_max_items", 1000);
    op_config.set("hbm_table.grow_limit", 1 << 20);
    RuntimeInfo rt(0, {0});
    HbmStorageOperator storage_op(op_config);
    std::unique_ptr<Storage> storage = storage_op.create_storage(rt, 0);
    auto* hst = static_cast<HbmShardStorage*>(storage.get());
    uint64_t in_use = 0, limit = 1;
    EXPECT(pshbm_device_memory(0, &in_use, &limit) == PSHBM_OK && in_use > 1000 * 64 * 4 && limit == 0);
    // room for the present arrays and a little more, not for arrays of 8,000 rows beside them
    initialize_device_memory(0, in_use + (1 << 20));
    std::vector<char> block;
    const size_t stride = 8 + 64 * 4;
    const int n = 5000;
    block.resize(n * stride);
    for (int k = 0; k < n; ++k) {
        const uint64_t key = 100 + k;
        std::memcpy(&block[k * stride], &key, 8);
        for (int c = 0; c < 64; ++c) {
            const float g = (float)(k % 7);
            std::memcpy(&block[k * stride + 8 + c * 4], &g, 4);
        }
    }
    auto push = [&]() {
        PSRequest req;
        req << (int32_t)1 << (int32_t)1 << (int32_t)0 << (int32_t)n;
        req.lazy().emplace_back(block.begin(), block.end());
        PSResponse resp;
        HbmSparsePushOperator push_op(op_config);
        push_op.apply_async_push_request(rt, req, storage.get(), nullptr, resp);
        Status status;
        resp >> status;
        return status;
    };
    Status st = push();
    EXPECT(st.IsOOM());
    EXPECT(hst->shard_size(0) == 0);
    uint64_t after = 0;
    EXPECT(pshbm_device_memory(0, &after, nullptr) == PSHBM_OK && after <= in_use + (1 << 20));
    initialize_device_memory(0, 0);
    st = push();
    EXPECT(st.ok());
    EXPECT(hst->shard_size(0) == (size_t)n);
    storage.reset();
    EXPECT(pshbm_device_memory(0, &after, nullptr) == PSHBM_OK && after < in_use);
}

// Sync to another cluster (operator/SyncOperator.h:102-266): what pushes wrote on the training side
// since the last sync arrives in the serving side's storage, block by block; a second walk finds
// nothing; later pushes travel with the next one.
static void test_sync() {
    struct ModPartitioner {
        int32_t partition(uint64_t key, int32_t global_shard_num) { return (int32_t)(key % (uint64_t)global_shard_num); }
    };
    Configure train_config;
    train_config.set("dim", 2);
    train_config.set("optimizer", "sum");
    train_config.set("hbm_table.expected_max_items", 1000);
    train_config.set("hbm_table.track_increment", 1);
    train_config.set("block_size", 64);
    Configure serve_config = train_config;
    serve_config.set("hbm_table.track_increment", 0);
    serve_config.set("hbm_table.expected_max_items", 100);   // grows as the synced items arrive
    serve_config.set("hbm_table.grow_limit", 4000);
    RuntimeInfo rt(0, {0, 1});
    HbmStorageOperator train_storage_op(train_config), serve_storage_op(serve_config);
    std::unique_ptr<Storage> train = train_storage_op.create_storage(rt, 0);
    std::unique_ptr<Storage> serve = serve_storage_op.create_storage(rt, 1);
    HbmSparsePushOperator push_op(train_config);
    HbmSparsePullOperator train_pull(train_config), serve_pull(serve_config);
    HbmSyncOperator<ModPartitioner> sync_op(train_config);

    auto push = [&](const std::vector<uint64_t>& keys, float arg) {
        PSRequest req = make_push_request(keys, std::vector<float>(keys.size(), arg));
        PSResponse resp;
        Status status;
        push_op.apply_async_push_request(rt, req, train.get(), nullptr, resp);
        resp >> status;
        EXPECT(status.ok());
    };
    auto sync = [&]() {   // returns the number of requests that carried items
        auto it = sync_op.incr_iterator(train.get());
        int sent = 0;
        while (true) {
            std::vector<PSRequest> reqs;
            Status st = sync_op.generate_sync_request(it.get(), rt, reqs);
            if (st.IsEmpty()) break;
            EXPECT(st.ok() && reqs.size() == 1);
            for (PSRequest& req : reqs) {
                PSResponse resp;
                Status status;
                sync_op.apply_sync_request(rt, req, serve.get(), resp);
                resp >> status;
                EXPECT(status.ok());
                ++sent;
            }
        }
        return sent;
    };
    std::vector<uint64_t> keys;
    for (uint64_t k = 0; k < 300; ++k) keys.push_back(k * 7 + 1);
    push(keys, 3.0f);   // [3, 1] per key
    EXPECT(sync() == 5);  // 300 items in blocks of 64
    bool ok;
    auto a = pull(train_pull, rt, train.get(), keys, &ok);
    EXPECT(ok);
    auto b = pull(serve_pull, rt, serve.get(), keys, &ok);
    EXPECT(ok);
    EXPECT(a == b);
    for (size_t i = 0; i < keys.size(); ++i) EXPECT(b[i * 2] == 3.0f && b[i * 2 + 1] == 1.0f);
    EXPECT(static_cast<HbmShardStorage*>(serve.get())->shard_size(0) + static_cast<HbmShardStorage*>(serve.get())->shard_size(1) == 300);
    EXPECT(sync() == 0);  // nothing was pushed since
    std::vector<uint64_t> some(keys.begin(), keys.begin() + 10), fresh{5000, 5001};
    push(some, 1.0f);
    push(fresh, 2.0f);
    EXPECT(sync() == 1);
    std::vector<uint64_t> all = keys;
    all.insert(all.end(), fresh.begin(), fresh.end());
    a = pull(train_pull, rt, train.get(), all, &ok);
    b = pull(serve_pull, rt, serve.get(), all, &ok);
    EXPECT(a == b);
    EXPECT(b[0] == 4.0f && b[1] == 2.0f && b[10 * 2] == 3.0f && b[300 * 2] == 2.0f && b[300 * 2 + 1] == 1.0f);
}

// The learning rate belongs to the push operator (pico-ps/operator/Operator.h:53-57): two operators
// registered with different rates push to one storage, each with its own.
static void test_operator_hyperparameters() {
    Configure storage_config;
    storage_config.set("dim", 2);
    storage_config.set("optimizer", "sgd");
    storage_config.set("lr", 0.5);
    storage_config.set("hbm_table.expected_max_items", 100);
    RuntimeInfo rt(0, {0, 1});
    HbmStorageOperator storage_op(storage_config);
    std::unique_ptr<Storage> storage = storage_op.create_storage(rt, 0);
    Configure slow = storage_config;
    slow.set("lr", 0.25);
    HbmSparsePushOperator push_fast(storage_config), push_slow(slow);
    HbmSparsePullOperator pull_op(storage_config);
    const std::vector<uint64_t> keys{10, 11, 12, 13};
    const std::vector<float> args{1.0f, 1.0f, 1.0f, 1.0f};  // gradient [arg, 1]
    auto push = [&](HbmSparsePushOperator& op) {
        PSRequest req = make_push_request(keys, args);
        PSResponse resp;
        Status status;
        op.apply_async_push_request(rt, req, storage.get(), nullptr, resp);
        resp >> status;
        EXPECT(status.ok());
    };
    push(push_fast);   // w = -0.5
    push(push_slow);   // w = -0.75
    push(push_fast);   // w = -1.25
    bool ok;
    auto v = pull(pull_op, rt, storage.get(), keys, &ok);
    EXPECT(ok);
    for (size_t i = 0; i < keys.size(); ++i) EXPECT(v[i * 2] == -1.25f && v[i * 2 + 1] == -1.25f);
}

// Several server threads push to the same shards at once (the reference runs apply_async_push_request
// on its c2s threads and serialises them per shard with shard.lock(), SparsePushOperator.h:220):
// two operators with different learning rates, a table that has to grow on the way. Each block is
// applied whole with the rate of the operator that brought it, so with gradients of 1 the weight of
// every key ends at -(pushes_fast * 0.5 + pushes_slow * 0.25) whatever the interleaving.
static void test_threaded_pushes() {
    Configure cfg;
    cfg.set("dim", 2);
    cfg.set("optimizer", "sgd");
    cfg.set("lr", 0.5);
    cfg.set("hbm_table.expected_max_items", 64);
    cfg.set("hbm_table.grow_limit", 4096);
    RuntimeInfo rt(0, {0, 1});
    HbmStorageOperator storage_op(cfg);
    std::unique_ptr<Storage> storage = storage_op.create_storage(rt, 0);
    Configure slow = cfg;
    slow.set("lr", 0.25);
    HbmSparsePushOperator push_fast(cfg), push_slow(slow);
    HbmSparsePullOperator pull_op(cfg);
    constexpr int THREADS = 6, ROUNDS = 8, KEYS = 600;
    std::vector<uint64_t> keys;
    std::vector<float> args;
    for (int k = 0; k < KEYS; ++k) {
        keys.push_back(1000 + k);
        args.push_back(1.0f);  // gradient [arg, 1]
    }
    std::atomic<int> failures{0};
    std::vector<std::thread> pool;
    for (int th = 0; th < THREADS; ++th)
        pool.emplace_back([&, th] {
            HbmSparsePushOperator& op = (th % 2 == 0) ? push_fast : push_slow;
            for (int r = 0; r < ROUNDS; ++r) {
                PSRequest req = make_push_request(keys, args);
                PSResponse resp;
                Status status;
                op.apply_async_push_request(rt, req, storage.get(), nullptr, resp);
                resp >> status;
                if (!status.ok()) ++failures;
            }
        });
    for (auto& t : pool) t.join();
    EXPECT(failures.load() == 0);
    bool ok;
    auto v = pull(pull_op, rt, storage.get(), keys, &ok);
    EXPECT(ok);
    const float want = -(THREADS / 2 * ROUNDS * 0.5f + THREADS / 2 * ROUNDS * 0.25f);
    for (size_t i = 0; i < keys.size(); ++i) EXPECT(v[i * 2] == want && v[i * 2 + 1] == want);
}

// Re-sharding with the library's key partitioner (HbmDefaultPartitioner: the shape of
// DefaultPartitioner<uint64_t>, common/Partitioner.h:43-61): two shards placed by partition(key, 2)
// become three; the generator hands out exactly the items whose partition changed, and the purge --
// one erase_if on the device per shard -- leaves exactly the others.
static void test_default_partitioner_purge() {
    Configure cfg;
    cfg.set("dim", 2);
    cfg.set("optimizer", "sum");
    cfg.set("hbm_table.expected_max_items", 4000);
    cfg.set("shuffle_block_items", 128);
    RuntimeInfo rt(0, {0, 1});
    HbmStorageOperator storage_op(cfg);
    std::unique_ptr<Storage> storage = storage_op.create_storage(rt, 0);
    HbmDefaultPartitioner part;
    HbmDirectPushOperator direct(cfg);
    std::vector<std::vector<Pair>> mine(2);
    constexpr uint64_t KEYS = 3000;
    for (uint64_t k = 1; k <= KEYS; ++k) {
        const uint64_t key = k * 0x9E3779B97F4A7C15ull;
        const int32_t sh = part.partition(key, 2);
        EXPECT(sh == 0 || sh == 1);
        mine[sh].push_back(Pair{key, {(float)k, 1.0f}});
    }
    EXPECT(mine[0].size() > KEYS / 3 && mine[1].size() > KEYS / 3);
    {
        PSRequest req;
        req << (int32_t)2 << (int32_t)1;
        for (int32_t sh = 0; sh < 2; ++sh) {
            req << sh << (int32_t)mine[sh].size();
            const char* p = reinterpret_cast<const char*>(mine[sh].data());
            req.lazy().emplace_back(p, p + mine[sh].size() * sizeof(Pair));
        }
        PSResponse resp;
        direct.apply_async_push_request(rt, req, storage.get(), nullptr, resp);
        Status s;
        resp >> s;
        EXPECT(s.ok());
    }
    HbmShuffleOperator<HbmDefaultPartitioner> shuffle_op(cfg);
    RuntimeInfo new_rt(0, {0, 1, 2});
    auto& st = *static_cast<HbmShardStorage*>(storage.get());
    size_t leaving = 0, expect_leaving = 0, expect_left[2] = {0, 0};
    for (int32_t sh = 0; sh < 2; ++sh)
        for (const Pair& it : mine[sh]) {
            if (part.partition(it.key, 3) != sh) ++expect_leaving;
            else ++expect_left[sh];
        }
    EXPECT(expect_leaving > KEYS / 6 && expect_leaving < KEYS / 2);  // about a third moves, all of it to shard 2
    for (int32_t sh = 0; sh < 2; ++sh) {
        auto gen = shuffle_op.lock_push_items_generator(new_rt, storage.get(), sh, false);
        std::vector<uint64_t> keys;
        std::vector<float> vals;
        while (gen->generate_push_items(keys, vals)) {}
        for (uint64_t key : keys) EXPECT(part.partition(key, 2) == sh && part.partition(key, 3) == 2);
        leaving += keys.size();
    }
    EXPECT(leaving == expect_leaving);
    for (int32_t sh = 0; sh < 2; ++sh) {
        PSRequest req;
        req << sh;
        PSResponse resp;
        shuffle_op.apply_purge_request(new_rt, req, storage.get(), resp);
        Status s;
        resp >> s;
        EXPECT(s.ok());
        EXPECT(st.shard_size(sh) == expect_left[sh]);
        std::vector<uint64_t> left(expect_left[sh] + 1);
        size_t got = 0;
        EXPECT(pshbm_iterate_keys(st.get(sh), 0, left.size(), left.data(), &got) == PSHBM_OK && got == expect_left[sh]);
        for (size_t i = 0; i < got; ++i) EXPECT(part.partition(left[i], 3) == sh);
    }
}

// hbm_table.init_range: a pull that misses answers the weights an insertion would store; a push
// of a new key takes its step from them (init_store_value, SparsePullOperator.h:217,307-310).
static void test_initial_weights() {
    Configure cfg;
    cfg.set("dim", 2);
    cfg.set("optimizer", "sgd");
    cfg.set("lr", 0.5);
    cfg.set("hbm_table.expected_max_items", 100);
    cfg.set("hbm_table.init_range", 0.125);
    RuntimeInfo rt(0, {0, 1});
    HbmStorageOperator storage_op(cfg);
    std::unique_ptr<Storage> storage = storage_op.create_storage(rt, 0);
    HbmSparsePushOperator push_op(cfg);
    HbmSparsePullOperator pull_op(cfg);
    const std::vector<uint64_t> keys{7, 8, 9};
    bool ok;
    auto v = pull(pull_op, rt, storage.get(), keys, &ok);
    EXPECT(ok);
    for (size_t i = 0; i < keys.size(); ++i)
        for (uint32_t c = 0; c < 2; ++c) {
            const float w = pshbm_init_weight(0.125f, keys[i], c);
            EXPECT(v[i * 2 + c] == w && w >= -0.125f && w < 0.125f);
        }
    EXPECT(v[0] != v[1] && v[0] != v[2]);
    PSRequest req = make_push_request(keys, std::vector<float>{2.0f, 2.0f, 2.0f});  // gradient [arg, 1]
    PSResponse resp;
    Status status;
    push_op.apply_async_push_request(rt, req, storage.get(), nullptr, resp);
    resp >> status;
    EXPECT(status.ok());
    v = pull(pull_op, rt, storage.get(), keys, &ok);
    EXPECT(ok);
    for (size_t i = 0; i < keys.size(); ++i) {
        EXPECT(v[i * 2] == pshbm_init_weight(0.125f, keys[i], 0) - 1.0f);
        EXPECT(v[i * 2 + 1] == pshbm_init_weight(0.125f, keys[i], 1) - 0.5f);
    }
}

int main(int argc, char** argv) {
    const std::string dir = argc > 1 ? argv[1] : "/tmp";
    Configure op_config;
    op_config.set("dim", 2);
    op_config.set("optimizer", "sum");
    op_config.set("hbm_table.expected_max_items", 1000);
    op_config.set("block_size", 100);  // ps_service_test.cpp:85
    RuntimeInfo rt(0, {0, 1});

    HbmStorageOperator storage_op(op_config);
    std::unique_ptr<Storage> storage = storage_op.create_storage(rt, 0);
    HbmSparsePushOperator push_op(op_config);
    std::unique_ptr<Storage> delta = push_op.create_delta_storage(rt);

    std::vector<uint64_t> all_keys;
    for (int rank = 0; rank < NUM_RANKS; ++rank) {
        std::vector<uint64_t> keys;
        std::vector<float> args;
        for (int k = rank * TEST_KEY_NUM; k < (rank + 1) * TEST_KEY_NUM; ++k) {
            keys.push_back(k);
            args.push_back((float)k);
            all_keys.push_back(k);
        }
        PSResponse resp;
        Status status;
        PSRequest a = make_push_request(keys, args);  // async_push, :104
        push_op.apply_async_push_request(rt, a, storage.get(), nullptr, resp);
        resp >> status;
        EXPECT(status.ok());
        for (int rep = 0; rep < (rank % 2 == 0 ? 2 : 1); ++rep) {  // sync_push, :106-111
            PSRequest s = make_push_request(keys, args);
            push_op.apply_sync_push_request(rt, s, storage.get(), resp);
            resp >> status;
            EXPECT(status.ok());
        }
    }
    // before the store only the asynchronous pushes are visible
    {
        bool ok;
        HbmSparsePullOperator pull_op(op_config);
        auto v = pull(pull_op, rt, storage.get(), all_keys, &ok);
        EXPECT(ok);
        for (size_t i = 0; i < all_keys.size(); ++i) EXPECT(v[i * 2] == (float)all_keys[i] && v[i * 2 + 1] == 1.0f);
    }
    for (int32_t shard = 0; shard < NUM_SHARDS; ++shard) {  // store, :120: one request per shard
        PSRequest req;
        req << shard;
        bool acked = false;
        push_op.apply_store_request(rt, req, delta.get(), storage.get(), nullptr, [&](PSResponse&& r) {
            Status s;
            r >> s;
            acked = s.ok();
        });
        EXPECT(acked);
    }
    auto total_size = [&](Storage* st) {
        PSRequest req;
        PSResponse resp;
        storage_op.apply_query_info_request(rt, req, st, resp);
        std::vector<StorageStatisticInfo> info;
        resp.archive() >> info;
        uint64_t n = 0;
        for (auto& i : info) {
            n += i.item_number;
            EXPECT(i.memory_usage > 0);
        }
        return n;
    };
    EXPECT(total_size(storage.get()) == (uint64_t)TEST_KEY_NUM * NUM_RANKS);  // :122

    // dump with file_number = 2 (:125-127): shard -> file by shard_id % file_number
    HbmDumpOperator<FileWriter> dump_op(op_config);
    std::vector<std::string> files;
    for (int32_t file_id = 0; file_id < 2; ++file_id) {
        PSRequest req;
        DumpArgs args{dir, 2};
        std::vector<int32_t> shard_ids;
        for (int32_t s = 0; s < NUM_SHARDS; ++s)
            if (s % 2 == file_id) shard_ids.push_back(s);
        req.archive() << args << file_id << shard_ids;
        PSResponse resp;
        dump_op.apply_request(rt, req, storage.get(), resp);
        Status s;
        resp >> s;
        EXPECT(s.ok());
        files.push_back(dir + "/model_0_" + std::to_string(file_id));
    }

    // a new storage, restore (no rehash, :150-156), clear, restore again
    std::unique_ptr<Storage> storage2 = storage_op.create_storage(rt, 1);
    HbmLoadOperator<FileReader> load_op(op_config);
    load_op.restore(files, rt, storage2.get(), partition);
    EXPECT(total_size(storage2.get()) == (uint64_t)TEST_KEY_NUM * NUM_RANKS);
    storage_op.clear_storage(storage2.get());
    EXPECT(total_size(storage2.get()) == 0);  // :153-154
    load_op.restore(files, rt, storage2.get(), partition);
    EXPECT(total_size(storage2.get()) == (uint64_t)TEST_KEY_NUM * NUM_RANKS);
    bool threw = false;  // restoring keys that are present aborts (LoadOperator.h:194,210)
    try {
        load_op.restore(files, rt, storage2.get(), partition);
    } catch (const std::logic_error&) {
        threw = true;
    }
    EXPECT(threw);

    // pulls, several times (:204-213): key * (2 + (rank even)); a missing key pulls 0 and is not inserted
    HbmSparsePullOperator pull_op(op_config);
    std::vector<uint64_t> q = all_keys;
    for (int i = 0; i < 10; ++i) q.push_back(TEST_KEY_NUM * NUM_RANKS + i);
    for (int rep = 0; rep < 3; ++rep) {
        for (Storage* st : {storage.get(), storage2.get()}) {
            bool ok;
            auto v = pull(pull_op, rt, st, q, &ok);
            EXPECT(ok);
            for (size_t i = 0; i < q.size(); ++i) {
                const uint64_t key = q[i];
                const int rank = (int)(key / TEST_KEY_NUM);
                const float count = key < (uint64_t)TEST_KEY_NUM * NUM_RANKS ? 2.0f + (rank % 2 == 0) : 0.0f;
                EXPECT(v[i * 2] == (float)key * count && v[i * 2 + 1] == count);
            }
        }
    }
    EXPECT(total_size(storage.get()) == (uint64_t)TEST_KEY_NUM * NUM_RANKS);

    // for-each over the restored storage: num = every record, and the merged columns
    // (ps_service_test.cpp:158-161; TestForEachOperator, TestOps.h:159-185); then erase_if(key % 2)
    // (TestEraseIfOperator, TestOps.h:138-150): half the records are left (:163-166) and an erased
    // key pulls 0 (:176-184)
    {
        HbmForEachOperator for_each_op(op_config);
        HbmEraseIfOperator erase_if_op(op_config);
        pshbm_predicate odd{};
        odd.struct_size = sizeof odd;
        odd.n_terms = 1;
        odd.term[0].column = PSHBM_COL_KEY;
        odd.term[0].cmp = PSHBM_CMP_MOD_EQ;
        odd.term[0].u = 2;
        odd.term[0].u2 = 1;
        erase_if_op.set_where(odd);
        auto sync_for_each = [&](Storage* st) {
            HbmForEachResult total;
            for (int32_t sh = 0; sh < NUM_SHARDS; ++sh) {
                PSRequest req;
                req << sh;
                PSResponse resp;
                for_each_op.apply_request(rt, req, st, resp);
                Status s;
                resp >> s;
                EXPECT(s.ok());
                HbmForEachResult one;
                resp.archive() >> one;
                total.merge(one);
            }
            return total;
        };
        double want_sum = 0, want_count = 0, even_sum = 0, even_count = 0;
        for (uint64_t key : all_keys) {
            const double count = 2.0 + ((key / TEST_KEY_NUM) % 2 == 0);
            want_sum += (double)key * count;
            want_count += count;
            if (key % 2 == 0) {
                even_sum += (double)key * count;
                even_count += count;
            }
        }
        HbmForEachResult all = sync_for_each(storage2.get());
        EXPECT(all.num == (int64_t)TEST_KEY_NUM * NUM_RANKS);
        EXPECT(all.sums.size() == 2 && all.sums[0] == want_sum && all.sums[1] == want_count);
        for (int32_t sh = 0; sh < NUM_SHARDS; ++sh) {
            PSRequest req;
            req << sh;
            PSResponse resp;
            erase_if_op.apply_request(rt, req, storage2.get(), resp);
            Status s;
            resp >> s;
            EXPECT(s.ok());
        }
        HbmForEachResult left = sync_for_each(storage2.get());
        EXPECT(left.num == (int64_t)TEST_KEY_NUM * NUM_RANKS / 2);
        EXPECT(left.sums[0] == even_sum && left.sums[1] == even_count);
        EXPECT(total_size(storage2.get()) == (uint64_t)TEST_KEY_NUM * NUM_RANKS / 2);
        bool ok;
        auto v = pull(pull_op, rt, storage2.get(), all_keys, &ok);
        EXPECT(ok);
        for (size_t i = 0; i < all_keys.size(); ++i) {
            const uint64_t key = all_keys[i];
            const float count = key % 2 ? 0.0f : 2.0f + ((key / TEST_KEY_NUM) % 2 == 0);
            EXPECT(v[i * 2] == (float)key * count && v[i * 2 + 1] == count);
        }
    }

    // coordinated restore of a shard from a replica, slice by slice (RestoreOperator.h:100-151), into
    // a storage that already holds some of the keys; then re-sharding from 2 to 3 shards: the items
    // that leave shard 0, and its purge (UpdateContextOperator.h:143-297)
    {
        struct ModPartitioner {
            int32_t partition(uint64_t key, int32_t global_shard_num) { return (int32_t)(key % (uint64_t)global_shard_num); }
        };
        std::unique_ptr<Storage> storage3 = storage_op.create_storage(rt, 2);
        {   // a few keys are there already, with other values: the restore must keep them
            HbmDirectPushOperator direct(op_config);
            std::vector<Pair> items = {{0, {-1.0f, -1.0f}}, {2, {-2.0f, -2.0f}}};
            PSRequest req;
            req << (int32_t)NUM_SHARDS << (int32_t)1;
            req << (int32_t)0 << (int32_t)items.size();
            const char* p = reinterpret_cast<const char*>(items.data());
            req.lazy().emplace_back(p, p + items.size() * sizeof(Pair));
            req << (int32_t)1 << (int32_t)0;
            PSResponse resp;
            direct.apply_async_push_request(rt, req, storage3.get(), nullptr, resp);
        }
        HbmRestoreOperator restore_op(op_config);
        for (int32_t sh = 0; sh < NUM_SHARDS; ++sh) {
            uint64_t offset = 0;
            for (bool finished = false; !finished;) {
                PSRequest req;
                req << (int32_t)0 << (int32_t)7 << offset << (uint64_t)37 << sh;
                PSResponse resp;
                restore_op.apply_coordinated_restore_request(req, storage.get(), resp);
                EXPECT(resp.error_code() == RpcErrorCodeType::SUCC);
                auto r = restore_op.apply_coordinated_restore_response(resp, storage3.get());
                finished = r.first;
                offset = r.second;
            }
        }
        EXPECT(total_size(storage3.get()) == (uint64_t)TEST_KEY_NUM * NUM_RANKS);
        bool ok;
        auto v3 = pull(pull_op, rt, storage3.get(), all_keys, &ok);
        for (size_t i = 0; i < all_keys.size(); ++i) {
            const uint64_t key = all_keys[i];
            const float count = 2.0f + ((key / TEST_KEY_NUM) % 2 == 0);
            if (key == 0 || key == 2)
                EXPECT(v3[i * 2] == -(float)(key / 2 + 1) && v3[i * 2 + 1] == -(float)(key / 2 + 1));
            else
                EXPECT(v3[i * 2] == (float)key * count && v3[i * 2 + 1] == count);
        }
        {   // a request for a shard that is not there
            PSRequest req;
            req << (int32_t)0 << (int32_t)7 << (uint64_t)0 << (uint64_t)10 << (int32_t)9;
            PSResponse resp;
            restore_op.apply_coordinated_restore_request(req, storage.get(), resp);
            EXPECT(resp.error_code() == RpcErrorCodeType::ELOGICERROR);
        }

        Configure shuffle_config = op_config;
        shuffle_config.set("shuffle_block_items", 64);
        HbmShuffleOperator<ModPartitioner> shuffle_op(shuffle_config);
        RuntimeInfo new_rt(0, {0, 1, 2});  // three shards now; this node keeps 0 and 1
        auto& st3 = *static_cast<HbmShardStorage*>(storage3.get());
        std::set<uint64_t> leaving;
        for (int32_t sh = 0; sh < NUM_SHARDS; ++sh) {
            auto gen = shuffle_op.lock_push_items_generator(new_rt, storage3.get(), sh, false);
            std::vector<uint64_t> keys;
            std::vector<float> vals;
            size_t blocks = 0;
            while (gen->generate_push_items(keys, vals)) ++blocks;
            EXPECT(blocks >= 1 && vals.size() == keys.size() * 2);
            for (size_t i = 0; i < keys.size(); ++i) {
                EXPECT(keys[i] % NUM_SHARDS == (uint64_t)sh && keys[i] % 3 != (uint64_t)sh);
                EXPECT(leaving.insert(keys[i]).second);
                if (keys[i] != 0 && keys[i] != 2) EXPECT(vals[i * 2 + 1] == 2.0f + ((keys[i] / TEST_KEY_NUM) % 2 == 0));
            }
        }
        size_t expect_leaving = 0;
        for (uint64_t key : all_keys) expect_leaving += (key % 3 != key % NUM_SHARDS);
        EXPECT(leaving.size() == expect_leaving);
        for (int32_t sh = 0; sh < NUM_SHARDS; ++sh) {
            PSRequest req;
            req << sh;
            PSResponse resp;
            shuffle_op.apply_purge_request(new_rt, req, storage3.get(), resp);
            Status s;
            resp >> s;
            EXPECT(s.ok());
        }
        EXPECT(total_size(storage3.get()) == all_keys.size() - expect_leaving);
        v3 = pull(pull_op, rt, storage3.get(), all_keys, &ok);
        for (size_t i = 0; i < all_keys.size(); ++i)
            if (leaving.count(all_keys[i])) EXPECT(v3[i * 2] == 0.0f && v3[i * 2 + 1] == 0.0f);
        (void)st3;
    }

    // direct push overwrites whole values (SparsePushOperator.h:557-562)
    {
        HbmDirectPushOperator direct(op_config);
        // (key 1 twice in one block: the later item stays, as after the reference's sequential safe_set)
        std::vector<Pair> items = {{0, {7.0f, 8.0f}}, {1, {-1.0f, -2.0f}}, {1000, {1.0f, 2.0f}}, {1, {9.0f, 10.0f}}};
        PSRequest req;
        req << (int32_t)NUM_SHARDS << (int32_t)1;
        for (int32_t s = 0; s < NUM_SHARDS; ++s) {
            std::vector<Pair> mine;
            for (auto& it : items)
                if (partition(it.key) == s) mine.push_back(it);
            req << s << (int32_t)mine.size();
            if (!mine.empty()) {
                const char* p = reinterpret_cast<const char*>(mine.data());
                req.lazy().emplace_back(p, p + mine.size() * sizeof(Pair));
            }
        }
        PSResponse resp;
        direct.apply_async_push_request(rt, req, storage.get(), nullptr, resp);
        Status s;
        resp >> s;
        EXPECT(s.ok());
        bool ok;
        auto v = pull(pull_op, rt, storage.get(), {0, 1, 1000, 2}, &ok);
        EXPECT(v[0] == 7.0f && v[1] == 8.0f && v[2] == 9.0f && v[3] == 10.0f && v[4] == 1.0f && v[5] == 2.0f);
        EXPECT(v[6] == 6.0f && v[7] == 3.0f);  // key 2, rank 0: 2 * 3
    }

    // a push that does not fit answers OOM and leaves the table as it was
    {
        std::vector<uint64_t> keys;
        std::vector<float> args;
        for (int k = 0; k < 2000; ++k) {
            keys.push_back(100000 + k);
            args.push_back(1.0f);
        }
        PSRequest req = make_push_request(keys, args);
        PSResponse resp;
        push_op.apply_async_push_request(rt, req, storage.get(), nullptr, resp);
        Status s;
        resp >> s;
        EXPECT(s.IsOOM() && resp.error_code() == RpcErrorCodeType::ELOGICERROR);
        EXPECT(total_size(storage.get()) == (uint64_t)TEST_KEY_NUM * NUM_RANKS + 1);
    }

    test_dense(dir);
    test_growth();
    test_operator_hyperparameters();
    test_threaded_pushes();
    test_default_partitioner_purge();
    test_initial_weights();
    test_memory_limit();
    test_sync();
    if (g_failed) {
        std::printf("FAILED: %d expectation(s)\n", g_failed);
        return 1;
    }
    std::printf("PASS test_hbm_operators\n");
    std::fflush(stdout);
    return 0;
}
