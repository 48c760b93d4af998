// mem.hpp — the executor's name -> tensor / argument store, HIP flavour.
//
// One Mem per process owns every tensor by name (executor/deepxcore/src/deepx/mem/mem.hpp:15-175;
// the CUDA twin executor/op-cuda/src/deepx/mem/mem_cuda.hpp).  Tensor storage is device memory
// obtained through the C ABI (dxh_pool_alloc / dxh_pool_free: freed blocks are handed out again; dxh_malloc / dxh_free
// with DEEPX_POOL=0), the counterpart of the alloc/free/copy
// function pointers the reference installs in Tensor<T> (executor/deepxcore/src/deepx/tensor.hpp:17-37,
// executor/op-cuda/src/deepx/tensorfunc/tensorlife_miaobyte.hpp:70-85).
#pragma once
#include <cstdlib>
#include <cstring>
#include <map>
#include <memory>
#include <stdexcept>
#include <string>
#include <unordered_map>
#include <variant>
#include <vector>
#include "../../include/dxhip.h"
#include "shape.hpp"

namespace deepx {

struct DxhError : std::runtime_error {
    int code;
    DxhError(int c, const std::string &what) : std::runtime_error(what + ": " + dxh_error_string(c)), code(c) {}
};
inline void dxh_check(int code, const char *what) { if (code != DXH_OK) throw DxhError(code, what); }

// Whether new tensors take their storage from the library's pool of freed blocks (default) or from the driver each time,
// as the reference does (DEEPX_POOL=0).  A pooled block can still be in use by launches made before it was freed, so
// the first launch on a new Tensor must be ordered behind them.  It is: everything runs on the NULL stream (replayed
// graphs on a blocking stream, which the NULL stream waits for) unless lines are spread over side streams, and there the
// `deltensor` that frees a block is a line for the default stream, before which the executor joins all streams.
inline bool &tensor_pool_enabled() {
    static bool on = [] { const char *e = std::getenv("DEEPX_POOL"); return !(e && !std::strcmp(e, "0")); }();
    return on;
}

// A device tensor: metadata + an owned HBM allocation.
struct Tensor {
    Shape shape;
    void *data = nullptr;
    bool pooled = false;
    // The tensor is new and reads as zeros by definition, but the fill has not been launched: the block holds whatever
    // its last owner left.  Nothing may launch a kernel that names the tensor before this is settled (Executor::settle).
    bool zero_pending = false;

    Tensor() = default;
    Tensor(const std::vector<int> &dims, Precision p) : shape(dims, p), pooled(tensor_pool_enabled()) {
        if (precision_bytes(p) == 0) throw std::invalid_argument("unsupported precision: " + precision_str(p));
        if (pooled) dxh_check(dxh_pool_alloc(&data, (size_t)shape.bytes()), "dxh_pool_alloc");
        else dxh_check(dxh_malloc(&data, (size_t)shape.bytes()), "dxh_malloc");
    }
    Tensor(const Tensor &) = delete;
    Tensor &operator=(const Tensor &) = delete;
    ~Tensor() {
        if (!data) return;
        if (pooled) dxh_pool_free(data);
        else dxh_free(data);
    }
    int dtype() const { return (int)shape.dtype; }  // Precision value == dxh_dtype value
    // launches the zero fill on `stream` (bool and f8 tensors fill as bytes) and clears zero_pending
    int fill_zero(void *stream) {
        zero_pending = false;
        const Precision p = shape.dtype;
        const int dt = (p == Precision::Float8E5M2 || p == Precision::Float8E4M3) ? (int)DXH_I8 : (int)p;
        return dxh_constant(dt, data, shape.size, dxh_scalar{0.0, 0}, stream);
    }
};

using ArgValue = std::variant<int32_t, int64_t, float, double, bool, std::string, std::vector<int32_t>,
                              std::vector<int64_t>, std::vector<float>, std::vector<double>, std::vector<std::string>>;

class Mem {
public:
    bool existstensor(const std::string &name) const { return tensors_.count(name) != 0; }
    std::shared_ptr<Tensor> gettensor(const std::string &name) const {
        auto it = tensors_.find(name);
        if (it == tensors_.end()) throw std::runtime_error("tensor not found: " + name);
        return it->second;
    }
    std::shared_ptr<Tensor> findtensor(const std::string &name) const {  // nullptr instead of throwing
        auto it = tensors_.find(name);
        return it == tensors_.end() ? nullptr : it->second;
    }
    // like MemBase::addtensor, an existing name is kept (mem.hpp:66-99) and reported
    bool addtensor(const std::string &name, std::shared_ptr<Tensor> t) { return tensors_.emplace(name, std::move(t)).second; }
    void delete_tensor(const std::string &name) { tensors_.erase(name); }
    void rename_tensor(const std::string &old_name, const std::string &new_name) {
        auto it = tensors_.find(old_name);
        if (it == tensors_.end()) throw std::runtime_error("tensor not found: " + old_name);
        auto t = it->second;
        tensors_.erase(it);
        tensors_[new_name] = t;
    }
    size_t tensor_count() const { return tensors_.size(); }

    bool existarg(const std::string &name) const { return args_.count(name) != 0; }
    void setarg(const std::string &name, ArgValue v) { args_[name] = std::move(v); }
    const ArgValue &getarg(const std::string &name) const {
        auto it = args_.find(name);
        if (it == args_.end()) throw std::runtime_error("arg not found: " + name);
        return it->second;
    }
    void clear() { tensors_.clear(); args_.clear(); }

    // Stream every op launches on: NULL (the default stream) except while the executor records or
    // replays a graph.  While recording nothing may allocate, so a workspace that would have to
    // grow aborts the recording instead.
    void *stream = nullptr;
    bool recording = false;
    // `newtensor` owes its zero fill to the first launch that names the tensor instead of making it at once (DEEPX_ZERO_AT_ALLOC=1
    // turns that off): the front allocates every result right before the op that overwrites it, and a fill of the result's
    // size costs about as much as a bandwidth-bound op itself.
    bool zero_later = [] { const char *e = std::getenv("DEEPX_ZERO_AT_ALLOC"); return !(e && !std::strcmp(e, "1")); }();

    // reusable device scratch for reductions and products (grown on demand, never shrunk).  Launches that may run
    // side by side on two streams must not share it: the executor names the scratch an op is to use (`scratch_of`,
    // NULL = the one of in-order execution, which recorded graphs pin) before it runs the op.
    void *scratch_of = nullptr;
    void *workspace(size_t bytes) {
        Scratch &w = scratch_[scratch_of];
        if (bytes > w.bytes) {
            if (recording) throw std::runtime_error("workspace would grow while recording a graph");
            if (w.ptr) { dxh_device_sync(); dxh_free(w.ptr); w.ptr = nullptr; w.bytes = 0; }
            size_t want = std::max<size_t>(bytes, (size_t)4 << 20);
            dxh_check(dxh_malloc(&w.ptr, want), "workspace dxh_malloc");
            w.bytes = want;
        }
        return w.ptr;
    }
    size_t workspace_bytes() const { auto it = scratch_.find(scratch_of); return it == scratch_.end() ? 0 : it->second.bytes; }
    const void *workspace_ptr() const { auto it = scratch_.find(scratch_of); return it == scratch_.end() ? nullptr : it->second.ptr; }
    ~Mem() {
        tensors_.clear();
        for (auto &kv : scratch_) if (kv.second.ptr) dxh_free(kv.second.ptr);
    }

private:
    std::unordered_map<std::string, std::shared_ptr<Tensor>> tensors_;
    std::unordered_map<std::string, ArgValue> args_;
    struct Scratch { void *ptr = nullptr; size_t bytes = 0; };
    std::unordered_map<void *, Scratch> scratch_;  // by `scratch_of`
};

}  // namespace deepx
