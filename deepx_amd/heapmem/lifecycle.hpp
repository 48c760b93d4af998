// lifecycle.hpp — consumes the `tensor_lifecycle` command list and owns the device memory of the
// heap tensors it created.
//
// Commands are the JSON objects of executor/heapmem-cuda/README.md:25-34,
//   {"op":"create|get|delete","name":"X","dtype":"f32","shape":[2,3],"device":0,"pid":123,"node":"n1"},
// parsed field by field like executor/heapmem-cuda/src/runtime/lifecycle.cpp:7-44 (the reference's
// extractor stops a "shape" array at its first comma; here the whole bracket is taken).
//   create  allocate device memory, export its IPC handle, write the hash (state ready, refcount 1);
//           an existing name gains a reference instead
//   get     refcount + 1 (the consumer opens the handle it reads from the hash)
//   delete  refcount - 1; at zero the hash goes and, if this process owns the memory, it is freed
#pragma once
#include <unistd.h>
#include <atomic>
#include <cctype>
#include <cstdlib>
#include <cstring>
#include <ctime>
#include <functional>
#include <map>
#include <string>
#include "../../include/dxhip.h"
#include "registry.hpp"

namespace deepx::heapmem {

// How the store gets device memory.  hip() is the product path (C ABI of libdxhip); host() backs
// tensors with calloc and an all-zero handle so that the control plane can be exercised on a
// machine without a GPU.
struct DeviceOps {
    std::function<int(void **, size_t)> alloc;
    std::function<int(void *)> release;
    std::function<int(const void *, void *)> export_handle;  // fills DXH_IPC_HANDLE_BYTES bytes

    static DeviceOps hip() {
        return {[](void **p, size_t n) { return dxh_malloc(p, n); }, [](void *p) { return dxh_free(p); },
                [](const void *p, void *h) { return dxh_ipc_export(p, h); }};
    }
    static DeviceOps host() {
        return {[](void **p, size_t n) { *p = std::calloc(n ? n : 1, 1); return *p ? 0 : 1; }, [](void *p) { std::free(p); return 0; },
                [](const void *, void *h) { std::memset(h, 0, DXH_IPC_HANDLE_BYTES); return 0; }};
    }
};

struct LifecycleCommand {
    std::string op, name, dtype, shape, node;
    long long device = 0, pid = 0;
};

// bytes per element for deepx dtype names and the short forms the reference's notes use
inline int dtype_bytes(const std::string &d) {
    if (d == "float64" || d == "f64" || d == "int64" || d == "i64") return 8;
    if (d == "float32" || d == "f32" || d == "int32" || d == "i32") return 4;
    if (d == "float16" || d == "f16" || d == "bfloat16" || d == "bf16" || d == "int16" || d == "i16") return 2;
    if (d == "int8" || d == "i8" || d == "bool" || d == "float8e5m2" || d == "float8e4m3") return 1;
    return 0;
}
// "[2,3,4]" or "[2 3 4]" -> element count; -1 when malformed
// Element count of "[2,3]" / "[2 3]"; -1 = malformed, -2 = the product does not fit (a count beyond
// kMaxElements is as good as overflow: no shared allocation may be that large).
constexpr long long kMaxElements = 1LL << 40;
inline long long shape_elements(const std::string &shape) {
    long long n = 1;
    bool any = false, in_number = false, too_big = false;
    long long cur = 0;
    auto fold = [&]() {
        if (cur != 0 && n > kMaxElements / cur) too_big = true; else n *= cur;
        cur = 0; in_number = false; any = true;
    };
    for (char c : shape) {
        if (std::isdigit((unsigned char)c)) {
            if (cur > kMaxElements) too_big = true; else cur = cur * 10 + (c - '0');
            in_number = true;
        }
        else if (c == ',' || c == ' ' || c == '[' || c == ']') { if (in_number) fold(); }
        else return -1;
    }
    if (in_number) fold();
    if (too_big) return n == 0 ? 0 : -2;  // a zero extent anywhere makes the tensor empty whatever the others say
    return any ? n : (shape.find('[') != std::string::npos ? 1 : -1);  // "[]" is a scalar
}
// A shared allocation stays under 2 GiB: larger IPC handles do not open on the target machines.
constexpr long long kMaxSharedBytes = (2LL << 30) - 1;
inline std::string to_hex(const unsigned char *bytes, size_t n) {
    static const char *digits = "0123456789abcdef";
    std::string s;
    for (size_t i = 0; i < n; ++i) { s += digits[bytes[i] >> 4]; s += digits[bytes[i] & 15]; }
    return s;
}

class LifecycleWorker {
public:
    LifecycleWorker(Registry *registry, const std::string &queue_key, DeviceOps ops)
        : registry_(registry), queue_key_(queue_key), ops_(std::move(ops)), running_(false) {}
    ~LifecycleWorker() { for (auto &kv : owned_) ops_.release(kv.second); }

    static std::string ExtractString(const std::string &json, const std::string &key) {
        auto pos = json.find("\"" + key + "\"");
        if (pos == std::string::npos) return "";
        pos = json.find(':', pos);
        if (pos == std::string::npos) return "";
        ++pos;
        while (pos < json.size() && std::isspace((unsigned char)json[pos])) ++pos;
        if (pos >= json.size()) return "";
        if (json[pos] == '"') {
            auto end = json.find('"', pos + 1);
            return end == std::string::npos ? "" : json.substr(pos + 1, end - pos - 1);
        }
        if (json[pos] == '[') {
            auto end = json.find(']', pos);
            return end == std::string::npos ? "" : json.substr(pos, end - pos + 1);
        }
        auto end = pos;
        while (end < json.size() && json[end] != ',' && json[end] != '}' && !std::isspace((unsigned char)json[end])) ++end;
        return json.substr(pos, end - pos);
    }
    static bool Parse(const std::string &json, LifecycleCommand &out) {
        out.op = ExtractString(json, "op");
        out.name = ExtractString(json, "name");
        out.dtype = ExtractString(json, "dtype");
        out.shape = ExtractString(json, "shape");
        out.node = ExtractString(json, "node");
        try {
            const std::string d = ExtractString(json, "device"), p = ExtractString(json, "pid");
            out.device = d.empty() ? 0 : std::stoll(d);
            out.pid = p.empty() ? 0 : std::stoll(p);
        } catch (const std::exception &) {
            return false;
        }
        return !out.op.empty() && !out.name.empty();
    }

    // returns an empty string on success, else why the command was not carried out
    std::string Handle(const LifecycleCommand &cmd) {
        if (cmd.op == "create") {
            TensorMeta existing;
            if (registry_->GetMeta(cmd.name, existing)) { registry_->RefInc(cmd.name); return ""; }
            const int es = dtype_bytes(cmd.dtype);
            const long long elements = shape_elements(cmd.shape);
            if (es == 0) return "unknown dtype: " + cmd.dtype;
            if (elements == -2 || (elements > 0 && elements > kMaxSharedBytes / es))
                return "tensor too large to share: " + cmd.shape + " " + cmd.dtype + " exceeds " + std::to_string(kMaxSharedBytes) + " bytes";
            if (elements < 0) return "malformed shape: " + cmd.shape;
            const long long bytes = elements * es;
            Release(cmd.name);  // memory of an earlier incarnation whose registry entry is gone
            void *ptr = nullptr;
            int rc = ops_.alloc(&ptr, (size_t)bytes);
            if (rc != 0 || !ptr) return std::string("allocation failed: ") + dxh_error_string(rc);
            unsigned char handle[DXH_IPC_HANDLE_BYTES];
            rc = ops_.export_handle(ptr, handle);
            if (rc != 0) { ops_.release(ptr); return std::string("handle export failed: ") + dxh_error_string(rc); }
            owned_[cmd.name] = ptr;
            registry_->CreateOrGet(cmd.name, cmd.dtype, cmd.shape, cmd.device, bytes, cmd.node, (long long)::getpid(),
                                   (long long)std::time(nullptr), to_hex(handle, sizeof handle));
            return "";
        }
        if (cmd.op == "get") return registry_->RefInc(cmd.name) < 0 ? "tensor not found: " + cmd.name : "";
        if (cmd.op == "delete") {
            const long long left = registry_->RefDec(cmd.name);
            if (left < 0) return "tensor not found: " + cmd.name;
            if (left == 0) Release(cmd.name);
            return "";
        }
        return "unknown op: " + cmd.op;
    }
    // one command from the list, waiting at most `timeout_seconds`; false when none arrived
    bool RunOnce(int timeout_seconds, std::string *error = nullptr) {
        std::string msg;
        if (!registry_->Client()->brpop(queue_key_, timeout_seconds, msg)) return false;
        LifecycleCommand cmd;
        std::string why = Parse(msg, cmd) ? Handle(cmd) : "malformed command: " + msg;
        if (error) *error = why;
        return true;
    }
    void RunLoop(int timeout_seconds) {
        running_.store(true);
        while (running_.load()) RunOnce(timeout_seconds);
    }
    void Stop() { running_.store(false); }

    // frees what a sweep removed from the registry
    long long Sweep(const std::string &node) {
        std::vector<std::string> removed;
        long long n = registry_->GcSweep(node, &removed);
        for (const auto &name : removed) Release(name);
        return n;
    }
    void *Pointer(const std::string &name) const {
        auto it = owned_.find(name);
        return it == owned_.end() ? nullptr : it->second;
    }
    size_t OwnedCount() const { return owned_.size(); }

private:
    void Release(const std::string &name) {
        auto it = owned_.find(name);
        if (it == owned_.end()) return;
        ops_.release(it->second);
        owned_.erase(it);
    }
    Registry *registry_;
    std::string queue_key_;
    DeviceOps ops_;
    std::atomic<bool> running_;
    std::map<std::string, void *> owned_;
};

}  // namespace deepx::heapmem
