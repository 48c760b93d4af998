// kv.hpp — the key-value operations the heap-tensor store needs, and an in-process backend.
//
// The reference's heap-tensor store keeps its state in Redis through a `RedisClient`
// (executor/heapmem-cuda/src/registry/registry.h:7,44; the class itself is not in the tree): one
// hash per tensor and one list of JSON commands.  This interface names exactly the Redis commands
// that are needed (HGETALL, HSET, HINCRBY, DEL, KEYS, LPUSH, BRPOP); `MemoryKV` implements them in
// the process, `RespKV` (resp.hpp) sends them to a Redis server.
#pragma once
#include <chrono>
#include <condition_variable>
#include <deque>
#include <map>
#include <mutex>
#include <string>
#include <vector>

namespace deepx::heapmem {

using Hash = std::map<std::string, std::string>;

class KV {
public:
    virtual ~KV() = default;
    virtual Hash hgetall(const std::string &key) = 0;                              // empty when the key does not exist
    virtual void hset(const std::string &key, const Hash &fields) = 0;
    virtual long long hincrby(const std::string &key, const std::string &field, long long by) = 0;
    virtual long long del(const std::string &key) = 0;                             // number of keys removed
    virtual std::vector<std::string> keys(const std::string &prefix) = 0;          // KEYS prefix*
    virtual void lpush(const std::string &list, const std::string &value) = 0;
    virtual bool brpop(const std::string &list, int timeout_seconds, std::string &value) = 0;
};

class MemoryKV : public KV {
public:
    Hash hgetall(const std::string &key) override {
        std::lock_guard<std::mutex> g(mu_);
        auto it = hashes_.find(key);
        return it == hashes_.end() ? Hash{} : it->second;
    }
    void hset(const std::string &key, const Hash &fields) override {
        std::lock_guard<std::mutex> g(mu_);
        for (const auto &kv : fields) hashes_[key][kv.first] = kv.second;
    }
    long long hincrby(const std::string &key, const std::string &field, long long by) override {
        std::lock_guard<std::mutex> g(mu_);
        std::string &v = hashes_[key][field];
        long long n = (v.empty() ? 0 : std::stoll(v)) + by;
        v = std::to_string(n);
        return n;
    }
    long long del(const std::string &key) override {
        std::lock_guard<std::mutex> g(mu_);
        return (long long)hashes_.erase(key);
    }
    std::vector<std::string> keys(const std::string &prefix) override {
        std::lock_guard<std::mutex> g(mu_);
        std::vector<std::string> out;
        for (const auto &kv : hashes_)
            if (kv.first.compare(0, prefix.size(), prefix) == 0) out.push_back(kv.first);
        return out;
    }
    void lpush(const std::string &list, const std::string &value) override {
        { std::lock_guard<std::mutex> g(mu_); lists_[list].push_front(value); }
        cv_.notify_all();
    }
    bool brpop(const std::string &list, int timeout_seconds, std::string &value) override {
        std::unique_lock<std::mutex> g(mu_);
        auto ready = [&] { auto it = lists_.find(list); return it != lists_.end() && !it->second.empty(); };
        if (!cv_.wait_for(g, std::chrono::seconds(timeout_seconds), ready)) return false;
        value = lists_[list].back();
        lists_[list].pop_back();
        return true;
    }

private:
    std::mutex mu_;
    std::condition_variable cv_;
    std::map<std::string, Hash> hashes_;
    std::map<std::string, std::deque<std::string>> lists_;
};

}  // namespace deepx::heapmem
