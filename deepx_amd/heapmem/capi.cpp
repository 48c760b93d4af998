// capi.cpp — libdxheap.so: the heap-tensor store behind a C ABI, for harnesses and for embedding it
// in another process.  backend: "memory" or "host:port" of a Redis server; device: "hip" or "host".
#include <cstring>
#include <memory>
#include <string>
#include "lifecycle.hpp"
#include "resp.hpp"

using namespace deepx::heapmem;

#define DXM_API extern "C" __attribute__((visibility("default")))

namespace {
struct Store {
    std::unique_ptr<KV> kv;
    std::unique_ptr<Registry> registry;
    std::unique_ptr<LifecycleWorker> worker;
    std::string last_error;
};
size_t copy_out(const std::string &s, char *buf, size_t buflen) {
    if (buf && buflen) {
        size_t n = s.size() < buflen - 1 ? s.size() : buflen - 1;
        std::memcpy(buf, s.data(), n);
        buf[n] = '\0';
    }
    return s.size();
}
}  // namespace

DXM_API void *dxm_create(const char *backend, const char *device) {
    try {
        auto s = std::make_unique<Store>();
        const std::string b = backend ? backend : "memory", d = device ? device : "hip";
        if (b == "memory") s->kv = std::make_unique<MemoryKV>();
        else {
            const size_t colon = b.rfind(':');
            if (colon == std::string::npos) return nullptr;
            s->kv = std::make_unique<RespKV>(b.substr(0, colon), std::atoi(b.c_str() + colon + 1));
        }
        s->registry = std::make_unique<Registry>(s->kv.get());
        s->worker = std::make_unique<LifecycleWorker>(s->registry.get(), "tensor_lifecycle", d == "host" ? DeviceOps::host() : DeviceOps::hip());
        return s.release();
    } catch (const std::exception &) {
        return nullptr;
    }
}
DXM_API void dxm_destroy(void *h) { delete static_cast<Store *>(h); }
// a compute process's side: put a command on the list
DXM_API int dxm_push(void *h, const char *json) {
    try { static_cast<Store *>(h)->kv->lpush("tensor_lifecycle", json ? json : ""); return 0; } catch (const std::exception &) { return 1; }
}
// the store's side: take one command (wait up to timeout_seconds); 1 = handled, 0 = none, -1 = handled with an error
DXM_API int dxm_run_once(void *h, int timeout_seconds) {
    auto *s = static_cast<Store *>(h);
    try {
        s->last_error.clear();
        if (!s->worker->RunOnce(timeout_seconds, &s->last_error)) return 0;
        return s->last_error.empty() ? 1 : -1;
    } catch (const std::exception &e) {
        s->last_error = e.what();
        return -1;
    }
}
DXM_API size_t dxm_last_error(void *h, char *out, size_t buflen) { return copy_out(static_cast<Store *>(h)->last_error, out, buflen); }
// the hash of a tensor as "field=value" lines in the field order of the reference's notes; empty when unknown
DXM_API size_t dxm_meta(void *h, const char *name, char *out, size_t buflen) {
    TensorMeta m;
    try {
        if (!static_cast<Store *>(h)->registry->GetMeta(name ? name : "", m)) return copy_out("", out, buflen);
    } catch (const std::exception &) {
        return copy_out("", out, buflen);
    }
    return copy_out("dtype=" + m.dtype + "\nshape=" + m.shape + "\nctime=" + std::to_string(m.ctime) + "\nnode=" + m.node +
                    "\ndevice=" + std::to_string(m.device) + "\nbytes=" + std::to_string(m.bytes) + "\nipc_handle=" + m.ipc_handle +
                    "\nrefcount=" + std::to_string(m.refcount) + "\nowner_pid=" + std::to_string(m.owner_pid) + "\nstate=" + m.state, out, buflen);
}
// device (or host) address of a tensor this store created; 0 when it does not own one by that name
DXM_API unsigned long long dxm_pointer(void *h, const char *name) {
    return (unsigned long long)(uintptr_t)static_cast<Store *>(h)->worker->Pointer(name ? name : "");
}
DXM_API long long dxm_owned(void *h) { return (long long)static_cast<Store *>(h)->worker->OwnedCount(); }
DXM_API long long dxm_sweep(void *h, const char *node) {
    try { return static_cast<Store *>(h)->worker->Sweep(node ? node : ""); } catch (const std::exception &) { return -1; }
}
