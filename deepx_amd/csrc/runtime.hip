// runtime.hip — device memory, copies, streams and events behind the C ABI.
// Replaces the cudaMalloc/cudaFree/cudaMemcpy calls of
// executor/op-cuda/src/deepx/tensorfunc/tensorlife_miaobyte.hpp:16-68.
#include "matmul_common.hpp"
#include "block_pool.hpp"
#include <cstdio>
#include <cstdlib>
#include <cstring>

using namespace dxh;

namespace dxh {
Tuning &tuning() {
    static Tuning t;
    return t;
}
}  // namespace dxh

namespace {

// A HIP call that fails leaves its code behind as the runtime's "last error" as well, where the next launch would find
// it and report it a second time as its own (the launchers ask hipGetLastError after every launch).  What is returned
// to the caller here is taken off there.
int reported(hipError_t e) {
    if (e != hipSuccess) (void)hipGetLastError();
    return (int)e;
}
int raw_alloc(void **p, size_t bytes) { return reported(hipMalloc(p, bytes)); }
int raw_free(void *p) { return reported(hipFree(p)); }

// One pool per device, made on first use and never destroyed: at process exit the runtime may be gone before a
// static destructor could hand the blocks back, and the driver reclaims them anyway.
// Kept bytes are capped at DXH_POOL_MAX_MB if set, else at half the device's memory.
BlockPool *pool_of_current_device(bool create) {
    static std::mutex mu;
    static std::map<int, BlockPool *> pools;
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess) { (void)hipGetLastError(); return nullptr; }
    std::lock_guard<std::mutex> lock(mu);
    auto it = pools.find(dev);
    if (it != pools.end()) return it->second;
    if (!create) return nullptr;
    size_t cap = 0;
    const char *e = std::getenv("DXH_POOL_MAX_MB");
    if (e && *e) {
        cap = (size_t)std::strtoull(e, nullptr, 10) << 20;
    } else {
        size_t free_b = 0, total_b = 0;
        if (hipMemGetInfo(&free_b, &total_b) != hipSuccess) { (void)hipGetLastError(); total_b = (size_t)16 << 30; }
        cap = total_b / 2;
    }
    BlockPool *p = new BlockPool(raw_alloc, raw_free, cap);
    pools[dev] = p;
    return p;
}

}  // namespace

extern "C" {

int dxh_version(void) { return DXH_ABI_VERSION; }

int dxh_tune(int knob, int64_t value) {
    Tuning &t = tuning();
    switch (knob) {
    case DXH_TUNE_NT_STORE_BYTES: t.nt_store_bytes = value; return DXH_OK;
    case DXH_TUNE_REDUCE_TARGET_BLOCKS: if (value < 1) return DXH_ERR_ARG; t.reduce_target_blocks = value; t.reduce_col_target_blocks = value; return DXH_OK;
    case DXH_TUNE_REDUCE_COL_MIN_ROWS: if (value < 1) return DXH_ERR_ARG; t.reduce_col_min_rows = value; return DXH_OK;
    case DXH_TUNE_REDUCE_COL_MAX_LANES:
        if (value != 4 && value != 8 && value != 16 && value != 32 && value != 64 && value != 128 && value != 256) return DXH_ERR_ARG;
        t.reduce_col_max_lanes = value;
        return DXH_OK;
    case DXH_TUNE_REDUCE_ROW_LOADS: if (value < 1 || value > 64) return DXH_ERR_ARG; t.reduce_row_loads = value; return DXH_OK;
    case DXH_TUNE_MATMUL_TILE: if (value < 0 || value > 15) return DXH_ERR_ARG; t.matmul_tile = value; return DXH_OK;
    case DXH_TUNE_MATMUL_SPLITK: if (value < 0 || value > 1024) return DXH_ERR_ARG; t.matmul_splitk = value; return DXH_OK;
    case DXH_TUNE_NT_LOAD: if (value < 0 || value > 2) return DXH_ERR_ARG; t.nt_load = value; return DXH_OK;
    case DXH_TUNE_SKINNY_PER_CU: if (value < 1 || value > 64) return DXH_ERR_ARG; t.skinny_per_cu = value; return DXH_OK;
    case DXH_TUNE_SKINNY_MIN_ROWS: if (value < 8) return DXH_ERR_ARG; t.skinny_min_rows = value; return DXH_OK;
    case DXH_TUNE_SKINNY_HALF: if (value < 0 || value > 1) return DXH_ERR_ARG; t.skinny_half = value; return DXH_OK;
    case DXH_TUNE_REDUCE_FUSED_FINISH: if (value < 0 || value > 1) return DXH_ERR_ARG; t.reduce_fused_finish = value; return DXH_OK;
    case DXH_TUNE_CHAIN_STATIC: if (value < 0 || value > 1) return DXH_ERR_ARG; t.chain_static = value; return DXH_OK;
    default: return DXH_ERR_ARG;
    }
}

const char *dxh_error_string(int code) {
    switch (code) {
    case DXH_OK: return "ok";
    case DXH_ERR_DTYPE: return "dtype not supported by this op";
    case DXH_ERR_ARG: return "invalid argument";
    case DXH_ERR_SHAPE: return "shape mismatch";
    case DXH_ERR_WORKSPACE: return "workspace missing or too small";
    case DXH_ERR_ALIGN: return "pointer not aligned to its element size";
    case DXH_ERR_TOO_LARGE: return "input needs more scratch than this entry point's fixed buffer holds";
    case DXH_ERR_NOT_READY: return "first use on this device is under stream capture: call dxh_set_device first";
    default: break;
    }
    if (code > 0) return hipGetErrorString((hipError_t)code);
    return "unknown error";
}

int dxh_device_count(int *count) {
    if (!count) return DXH_ERR_ARG;
    hipError_t e = hipGetDeviceCount(count);
    if (e != hipSuccess) { *count = 0; (void)hipGetLastError(); }
    return reported(e);
}
int dxh_set_device(int device) {
    hipError_t e = hipSetDevice(device);
    if (e == hipSuccess) { dxh::reduce_device_init(); dxh::chain_device_init(); }
    return reported(e);
}
int dxh_device_name(char *buf, size_t buflen) {
    if (!buf || buflen == 0) return DXH_ERR_ARG;
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return reported(e);
    hipDeviceProp_t prop;
    e = hipGetDeviceProperties(&prop, dev);
    if (e != hipSuccess) return reported(e);
    snprintf(buf, buflen, "%s %s cus=%d clock_khz=%d", prop.name, prop.gcnArchName, prop.multiProcessorCount, prop.clockRate);
    return DXH_OK;
}

int dxh_malloc(void **ptr, size_t bytes) {
    if (!ptr) return DXH_ERR_ARG;
    *ptr = nullptr;
    if (bytes == 0) bytes = 1;  // a zero-element tensor still owns a distinct pointer
    hipError_t e = hipMalloc(ptr, bytes);
    if (e == hipErrorOutOfMemory) {  // blocks kept for reuse may be what is in the way
        (void)hipGetLastError();
        BlockPool *pool = pool_of_current_device(false);
        if (pool && pool->trim(0) > 0) e = hipMalloc(ptr, bytes);
    }
    return reported(e);
}
int dxh_free(void *ptr) { return ptr ? reported(hipFree(ptr)) : DXH_OK; }

int dxh_pool_alloc(void **ptr, size_t bytes) {
    if (!ptr) return DXH_ERR_ARG;
    *ptr = nullptr;
    BlockPool *pool = pool_of_current_device(true);
    if (!pool) return DXH_ERR_ARG;
    const int rc = pool->alloc(ptr, bytes);
    if (rc > 0) (void)hipGetLastError();
    return rc < 0 ? DXH_ERR_ARG : rc;
}
int dxh_pool_free(void *ptr) {
    if (!ptr) return DXH_OK;
    BlockPool *pool = pool_of_current_device(false);
    if (!pool) return DXH_ERR_ARG;
    const int rc = pool->free(ptr);
    return rc < 0 ? DXH_ERR_ARG : rc;
}
int dxh_pool_trim(size_t keep_bytes, size_t *released) {
    BlockPool *pool = pool_of_current_device(false);
    const size_t gone = pool ? pool->trim(keep_bytes) : 0;
    if (released) *released = gone;
    return DXH_OK;
}
int dxh_pool_limit(size_t max_kept_bytes) {
    BlockPool *pool = pool_of_current_device(true);
    if (!pool) return DXH_ERR_ARG;
    pool->set_max_kept(max_kept_bytes);
    return DXH_OK;
}
int dxh_pool_stats(dxh_pool_stats_t *out) {
    if (!out) return DXH_ERR_ARG;
    BlockPool *pool = pool_of_current_device(false);
    const BlockPool::Stats s = pool ? pool->stats() : BlockPool::Stats();
    out->hits = s.hits; out->misses = s.misses; out->kept = s.kept; out->released = s.released;
    out->kept_bytes = s.kept_bytes; out->kept_blocks = s.kept_blocks; out->live_bytes = s.live_bytes; out->live_blocks = s.live_blocks;
    return DXH_OK;
}

int dxh_memcpy_h2d(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return DXH_OK;
    if (!dst || !src) return DXH_ERR_ARG;
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyHostToDevice, as_stream(stream));
    if (e != hipSuccess) return reported(e);
    return reported(hipStreamSynchronize(as_stream(stream)));  // pageable source must stay valid
}
int dxh_memcpy_d2h(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return DXH_OK;
    if (!dst || !src) return DXH_ERR_ARG;
    hipError_t e = hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToHost, as_stream(stream));
    if (e != hipSuccess) return reported(e);
    return reported(hipStreamSynchronize(as_stream(stream)));
}
int dxh_memcpy_d2d(void *dst, const void *src, size_t bytes, void *stream) {
    if (bytes == 0) return DXH_OK;
    if (!dst || !src) return DXH_ERR_ARG;
    return reported(hipMemcpyAsync(dst, src, bytes, hipMemcpyDeviceToDevice, as_stream(stream)));
}

int dxh_stream_create(void **stream) {
    if (!stream) return DXH_ERR_ARG;
    hipStream_t s = nullptr;
    hipError_t e = hipStreamCreate(&s);  // default priority only
    *stream = (void *)s;
    return reported(e);
}
int dxh_stream_destroy(void *stream) {
    if (!stream) return DXH_OK;
    dxh::reduce_stream_release(as_stream(stream));
    return reported(hipStreamDestroy(as_stream(stream)));
}
int dxh_stream_sync(void *stream) { return reported(hipStreamSynchronize(as_stream(stream))); }
int dxh_device_sync(void) { return reported(hipDeviceSynchronize()); }

int dxh_event_create(void **event) {
    if (!event) return DXH_ERR_ARG;
    hipEvent_t ev = nullptr;
    hipError_t e = hipEventCreate(&ev);
    *event = (void *)ev;
    return reported(e);
}
int dxh_event_destroy(void *event) { return event ? reported(hipEventDestroy((hipEvent_t)event)) : DXH_OK; }
int dxh_event_record(void *event, void *stream) {
    if (!event) return DXH_ERR_ARG;
    return reported(hipEventRecord((hipEvent_t)event, as_stream(stream)));
}
int dxh_stream_wait_event(void *stream, void *event) {
    if (!event) return DXH_ERR_ARG;
    return reported(hipStreamWaitEvent(as_stream(stream), (hipEvent_t)event, 0));
}
int dxh_event_sync(void *event) {
    if (!event) return DXH_ERR_ARG;
    return reported(hipEventSynchronize((hipEvent_t)event));
}
int dxh_event_elapsed_ms(void *start, void *stop, float *ms) {
    if (!start || !stop || !ms) return DXH_ERR_ARG;
    return reported(hipEventElapsedTime(ms, (hipEvent_t)start, (hipEvent_t)stop));
}

static_assert(sizeof(hipIpcMemHandle_t) == DXH_IPC_HANDLE_BYTES, "handle size is part of the ABI");
int dxh_ipc_export(const void *ptr, void *handle) {
    if (!ptr || !handle) return DXH_ERR_ARG;
    hipIpcMemHandle_t h;
    hipError_t e = hipIpcGetMemHandle(&h, const_cast<void *>(ptr));
    if (e != hipSuccess) return reported(e);
    std::memcpy(handle, &h, sizeof h);
    return DXH_OK;
}
int dxh_ipc_open(const void *handle, void **ptr) {
    if (!handle || !ptr) return DXH_ERR_ARG;
    *ptr = nullptr;
    hipIpcMemHandle_t h;
    std::memcpy(&h, handle, sizeof h);
    return reported(hipIpcOpenMemHandle(ptr, h, hipIpcMemLazyEnablePeerAccess));
}
int dxh_ipc_close(void *ptr) { return ptr ? reported(hipIpcCloseMemHandle(ptr)) : DXH_OK; }

int dxh_graph_begin_capture(void *stream) {
    if (!stream) return DXH_ERR_ARG;  // the NULL stream cannot be captured
    return reported(hipStreamBeginCapture(as_stream(stream), hipStreamCaptureModeThreadLocal));
}
int dxh_graph_end_capture(void *stream, void **graph_exec) {
    if (!stream || !graph_exec) return DXH_ERR_ARG;
    *graph_exec = nullptr;
    hipGraph_t graph = nullptr;
    hipError_t e = hipStreamEndCapture(as_stream(stream), &graph);
    if (e != hipSuccess || !graph) {
        (void)hipGetLastError();
        dxh::finish_capture_ended(as_stream(stream), nullptr);
        return e != hipSuccess ? (int)e : DXH_ERR_ARG;
    }
    hipGraphExec_t exec = nullptr;
    e = hipGraphInstantiate(&exec, graph, nullptr, nullptr, 0);
    (void)hipGraphDestroy(graph);
    if (e != hipSuccess) { dxh::finish_capture_ended(as_stream(stream), nullptr); return reported(e); }
    // the in-launch counters its recorded launches took stay with the graph until dxh_graph_destroy
    dxh::finish_capture_ended(as_stream(stream), (const void *)exec);
    *graph_exec = (void *)exec;
    return DXH_OK;
}
int dxh_graph_launch(void *graph_exec, void *stream) {
    if (!graph_exec || !stream) return DXH_ERR_ARG;
    return reported(hipGraphLaunch((hipGraphExec_t)graph_exec, as_stream(stream)));
}
int dxh_graph_destroy(void *graph_exec) {
    if (!graph_exec) return DXH_OK;
    const hipError_t e = hipGraphExecDestroy((hipGraphExec_t)graph_exec);
    dxh::finish_graph_destroyed(graph_exec);
    return reported(e);
}
int dxh_graph_counter_stats(int64_t *in_use, int64_t *capacity) {
    if (!in_use || !capacity) return DXH_ERR_ARG;
    dxh::finish_capture_stats(in_use, capacity);
    return DXH_OK;
}

}  // extern "C"
