// deepx-heapmem-hip — the heap-tensor store process: connects to Redis, sweeps what a previous
// instance left behind on this node, then serves the `tensor_lifecycle` list
// (executor/heapmem-cuda/README.md:24-34).  DEEPX_REDIS=host:port (default 127.0.0.1:6379),
// DEEPX_NODE (default the host name), DEEPX_DEVICE (default 0).
#include <csignal>
#include <cstdlib>
#include <iostream>
#include "lifecycle.hpp"
#include "resp.hpp"

using namespace deepx::heapmem;

static LifecycleWorker *g_worker = nullptr;
static void on_signal(int) { if (g_worker) g_worker->Stop(); }

int main() {
    std::string target = std::getenv("DEEPX_REDIS") ? std::getenv("DEEPX_REDIS") : "127.0.0.1:6379";
    const size_t colon = target.rfind(':');
    const std::string host = colon == std::string::npos ? target : target.substr(0, colon);
    const int port = colon == std::string::npos ? 6379 : std::atoi(target.c_str() + colon + 1);
    char hostname[256] = "node";
    gethostname(hostname, sizeof hostname - 1);
    const std::string node = std::getenv("DEEPX_NODE") ? std::getenv("DEEPX_NODE") : hostname;
    int count = 0;
    if (dxh_device_count(&count) != DXH_OK || count == 0) { std::cerr << "no HIP device\n"; return 1; }
    if (dxh_set_device(std::getenv("DEEPX_DEVICE") ? std::atoi(std::getenv("DEEPX_DEVICE")) : 0) != DXH_OK) { std::cerr << "cannot select device\n"; return 1; }
    try {
        RespKV kv(host, port);
        Registry registry(&kv);
        LifecycleWorker worker(&registry, "tensor_lifecycle", DeviceOps::hip());
        g_worker = &worker;
        std::signal(SIGINT, on_signal);
        std::signal(SIGTERM, on_signal);
        std::cout << "heapmem-hip: node " << node << ", swept " << worker.Sweep(node) << " stale tensors" << std::endl;
        worker.RunLoop(1);
    } catch (const std::exception &e) {
        std::cerr << e.what() << std::endl;
        return 1;
    }
    return 0;
}
