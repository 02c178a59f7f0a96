// Stand-ins for the prpc / pico-ps types that the operator signatures of this path name.
//
// pico-ps compiles against prpc (pico-core), which is not available to this repository. So that
// the operator mirror in hbm_ops.h can be compiled and tested on its own, this header supplies the
// few types those signatures use, with the same names, members and byte layout on the wire:
// BinaryArchive / PSRequest / PSResponse (pico-ps/common/message.h:65-204), Status
// (pico-ps/common/Status.h:15-197), RuntimeInfo::local_shards / node_id
// (pico-ps/service/TableDescriptor.h:180-228), Configure (prpc's YAML tree, reduced to a flat map),
// Storage (pico-ps/storage/Storage.h:24-47), StorageStatisticInfo
// (pico-ps/operator/StorageOperator.h:27-38). With a prpc checkout, include the pico-ps headers
// instead of this file and build hbm_ops.h against the real types; nothing else changes.
#pragma once

#include <cstdint>
#include <cstring>
#include <deque>
#include <map>
#include <set>
#include <stdexcept>
#include <string>
#include <type_traits>
#include <vector>

namespace pshbm_host {

// Raw little-endian byte stream: trivially copyable values are memcpy'd (message.h:177-204).
class BinaryArchive {
public:
    BinaryArchive() = default;
    explicit BinaryArchive(std::vector<char> bytes) : _buf(std::move(bytes)) {}
    template <class T>
    std::enable_if_t<std::is_trivially_copyable<T>::value, BinaryArchive&> operator<<(const T& v) {
        const char* p = reinterpret_cast<const char*>(&v);
        _buf.insert(_buf.end(), p, p + sizeof(T));
        return *this;
    }
    template <class T>
    std::enable_if_t<std::is_trivially_copyable<T>::value, BinaryArchive&> operator>>(T& v) {
        if (_pos + sizeof(T) > _buf.size()) throw std::runtime_error("archive exhausted");
        std::memcpy(&v, _buf.data() + _pos, sizeof(T));
        _pos += sizeof(T);
        return *this;
    }
    BinaryArchive& operator<<(const std::string& s) {
        *this << (uint64_t)s.size();
        _buf.insert(_buf.end(), s.begin(), s.end());
        return *this;
    }
    BinaryArchive& operator>>(std::string& s) {
        uint64_t n;
        *this >> n;
        if (_pos + n > _buf.size()) throw std::runtime_error("archive exhausted");
        s.assign(_buf.data() + _pos, n);
        _pos += n;
        return *this;
    }
    template <class T>
    BinaryArchive& operator<<(const std::vector<T>& v) {
        *this << (uint64_t)v.size();
        for (const T& x : v) *this << x;
        return *this;
    }
    template <class T>
    BinaryArchive& operator>>(std::vector<T>& v) {
        uint64_t n;
        *this >> n;
        v.resize(n);
        for (T& x : v) *this >> x;
        return *this;
    }
    void write_raw(const void* p, size_t n) {
        const char* c = static_cast<const char*>(p);
        _buf.insert(_buf.end(), c, c + n);
    }
    const char* cursor() const { return _buf.data() + _pos; }
    size_t readable() const { return _buf.size() - _pos; }
    void advance(size_t n) { _pos += n; }
    bool is_exhausted() const { return _pos == _buf.size(); }
    std::vector<char>& buffer() { return _buf; }
    size_t size() const { return _buf.size(); }
    void clear() {
        _buf.clear();
        _pos = 0;
    }

private:
    std::vector<char> _buf;
    size_t _pos = 0;
};

// pico-ps/common/Status.h
enum class StatusCode : int32_t { OK = 0, INVALID_CONFIG = 1, INVALID_ID = 2, OUT_OF_MEMORY = 3, NO_REPLICA = 9,
                                  ERROR = 10, FATAL = 11, EMPTY = 12 };
class Status {
public:
    Status() = default;
    static Status OOM(const std::string& m) { return Status(StatusCode::OUT_OF_MEMORY, m); }
    static Status Error(const std::string& m) { return Status(StatusCode::ERROR, m); }
    static Status Fatal(const std::string& m) { return Status(StatusCode::FATAL, m); }
    static Status InvalidConfig(const std::string& m) { return Status(StatusCode::INVALID_CONFIG, m); }
    static Status InvalidID(const std::string& m) { return Status(StatusCode::INVALID_ID, m); }
    static Status NoReplica(const std::string& m) { return Status(StatusCode::NO_REPLICA, m); }
    static Status Empty(const std::string& m) { return Status(StatusCode::EMPTY, m); }
    bool IsEmpty() const { return _code == StatusCode::EMPTY; }
    bool ok() const { return _code == StatusCode::OK; }
    bool IsOOM() const { return _code == StatusCode::OUT_OF_MEMORY; }
    StatusCode code() const { return _code; }
    const std::string& msg() const { return _msg; }
    friend BinaryArchive& operator<<(BinaryArchive& ar, const Status& s) { return ar << (int32_t)s._code << s._msg; }
    friend BinaryArchive& operator>>(BinaryArchive& ar, Status& s) {
        int32_t c;
        ar >> c >> s._msg;
        s._code = (StatusCode)c;
        return ar;
    }

private:
    Status(StatusCode c, std::string m) : _code(c), _msg(std::move(m)) {}
    StatusCode _code = StatusCode::OK;
    std::string _msg;
};

enum class RpcErrorCodeType : int32_t { SUCC = 0, ELOGICERROR = 1 };

// A message: an archive plus "lazy" blocks that travel beside it without being copied into it
// (message.h:104-109, 218-236; vector_rpc_view :276-294).
class PSMessage {
public:
    BinaryArchive& archive() { return _ar; }
    std::deque<std::vector<char>>& lazy() { return _lazy; }
    template <class T>
    PSMessage& operator<<(const T& v) {
        _ar << v;
        return *this;
    }
    template <class T>
    PSMessage& operator>>(T& v) {
        _ar >> v;
        return *this;
    }
    void set_error_code(RpcErrorCodeType c) { _err = c; }
    RpcErrorCodeType error_code() const { return _err; }

private:
    BinaryArchive _ar;
    std::deque<std::vector<char>> _lazy;
    RpcErrorCodeType _err = RpcErrorCodeType::SUCC;
};
class PSRequest : public PSMessage {};
class PSResponse : public PSMessage {
public:
    PSResponse() = default;
    explicit PSResponse(PSRequest&) {}
    PSResponse& rpc_response() { return *this; }
};

// ps_serialize / ps_deserialize of a lazy block without compression (message.h:218-236)
inline void ps_serialize(std::deque<std::vector<char>>& lazy, std::vector<char>&& block) { lazy.push_back(std::move(block)); }
inline void ps_deserialize(std::deque<std::vector<char>>& lazy, std::vector<char>& block) {
    if (lazy.empty()) throw std::runtime_error("no lazy block");
    block = std::move(lazy.front());
    lazy.pop_front();
}

class RuntimeInfo {
public:
    RuntimeInfo(int32_t node_id, std::set<int32_t> shards) : _node(node_id), _shards(std::move(shards)) {}
    const std::set<int32_t>& local_shards() const { return _shards; }
    int32_t node_id() const { return _node; }
    int32_t global_shard_num() const { return (int32_t)_shards.size(); }
    // node -> the shards it holds (TableDescriptor.h:180-228); the stand-in knows one node
    std::map<int32_t, std::vector<int32_t>> nodes() const {
        return {{_node, std::vector<int32_t>(_shards.begin(), _shards.end())}};
    }

private:
    int32_t _node;
    std::set<int32_t> _shards;
};

// prpc's Configure is a YAML tree; the operators of this path only read scalars of `op_config`.
class Configure {
public:
    bool has(const std::string& k) const { return _kv.count(k) != 0; }
    void set(const std::string& k, const std::string& v) { _kv[k] = v; }
    void set(const std::string& k, double v) { _kv[k] = std::to_string(v); }
    double number(const std::string& k, double dflt) const { return has(k) ? std::stod(_kv.at(k)) : dflt; }
    std::string str(const std::string& k, const std::string& dflt) const { return has(k) ? _kv.at(k) : dflt; }

private:
    std::map<std::string, std::string> _kv;
};

class Storage {
public:
    virtual ~Storage() = default;
    virtual bool need_remote_restore() { return false; }  // Storage.h:29-40
};

struct StorageStatisticInfo {  // StorageOperator.h:27-38
    int32_t node_id;
    int32_t shard_id;
    uint64_t item_number;
    uint64_t memory_usage;
};

#define PSHBM_SCHECK(cond, msg)                                         \
    do {                                                                \
        if (!(cond)) throw std::logic_error(std::string("SCHECK: ") + (msg)); \
    } while (0)

}  // namespace pshbm_host
