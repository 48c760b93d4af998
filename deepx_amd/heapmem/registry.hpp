// registry.hpp — name -> heap-tensor metadata, one hash `tensor:<name>` per tensor.
//
// Same fields and entry points as the reference's Registry
// (executor/heapmem-cuda/src/registry/registry.h:11-44, registry.cpp:11-86; field list
// executor/heapmem-cuda/README.md:13-22).  The reference delegates create_or_get / ref_inc /
// ref_dec / gc_sweep to Lua scripts that are not in its tree (registry.cpp:42,48,55,62); here they
// are written out over plain hash commands.  The store process is the only writer of these hashes
// (compute processes push commands on the list and read), so no server-side script is needed for
// atomicity.
#pragma once
#include <csignal>
#include <string>
#include <vector>
#include "kv.hpp"

namespace deepx::heapmem {

struct TensorMeta {
    std::string dtype, shape, node, ipc_handle, state;
    long long device = 0, bytes = 0, refcount = 0, owner_pid = 0, ctime = 0;
};

class Registry {
public:
    explicit Registry(KV *client) : client_(client) {}

    static std::string Key(const std::string &name) { return "tensor:" + name; }

    // A new name is written with refcount 1 and state "ready"; an existing one gains a reference.
    // Either way the stored IPC handle comes back.  `created` tells the two cases apart.
    std::string CreateOrGet(const std::string &name, const std::string &dtype, const std::string &shape, long long device,
                            long long bytes, const std::string &node, long long pid, long long ctime,
                            const std::string &ipc_handle, bool *created = nullptr) {
        Hash h = client_->hgetall(Key(name));
        if (!h.empty()) {
            client_->hincrby(Key(name), "refcount", 1);
            if (created) *created = false;
            return h["ipc_handle"];
        }
        client_->hset(Key(name), {{"dtype", dtype}, {"shape", shape}, {"device", std::to_string(device)},
                                  {"bytes", std::to_string(bytes)}, {"node", node}, {"owner_pid", std::to_string(pid)},
                                  {"ctime", std::to_string(ctime)}, {"ipc_handle", ipc_handle}, {"refcount", "1"},
                                  {"state", "ready"}});
        if (created) *created = true;
        return ipc_handle;
    }
    // -1 when the tensor does not exist
    long long RefInc(const std::string &name) {
        if (client_->hgetall(Key(name)).empty()) return -1;
        return client_->hincrby(Key(name), "refcount", 1);
    }
    // new count; at zero the hash is removed (the owner then frees the memory); -1 when unknown
    long long RefDec(const std::string &name) {
        if (client_->hgetall(Key(name)).empty()) return -1;
        long long n = client_->hincrby(Key(name), "refcount", -1);
        if (n <= 0) { client_->del(Key(name)); return 0; }
        return n;
    }
    // removes every tensor of `node` that nobody references or whose owning process is gone;
    // returns how many, and their names through `removed`
    long long GcSweep(const std::string &node, std::vector<std::string> *removed = nullptr) {
        long long count = 0;
        for (const std::string &key : client_->keys("tensor:")) {
            Hash h = client_->hgetall(key);
            if (h.empty() || h["node"] != node) continue;
            const long long refs = h.count("refcount") ? std::stoll(h["refcount"]) : 0;
            const long long pid = h.count("owner_pid") ? std::stoll(h["owner_pid"]) : 0;
            const bool owner_gone = pid > 0 && ::kill((pid_t)pid, 0) != 0;
            if (refs > 0 && !owner_gone) continue;
            client_->del(key);
            if (removed) removed->push_back(key.substr(7));
            ++count;
        }
        return count;
    }
    bool GetMeta(const std::string &name, TensorMeta &out) const {
        Hash map = client_->hgetall(Key(name));
        if (map.empty()) return false;
        out.dtype = map["dtype"]; out.shape = map["shape"]; out.node = map["node"];
        out.ipc_handle = map["ipc_handle"]; out.state = map["state"];
        auto num = [&](const char *k) { return map.count(k) && !map[k].empty() ? std::stoll(map[k]) : 0LL; };
        out.device = num("device"); out.bytes = num("bytes"); out.refcount = num("refcount");
        out.owner_pid = num("owner_pid"); out.ctime = num("ctime");
        return true;
    }
    KV *Client() const { return client_; }

private:
    KV *client_;
};

}  // namespace deepx::heapmem
