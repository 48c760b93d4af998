// deepx-executor-hip — the MI355X executor process: a drop-in for executor/op-cuda's and
// executor/op-ompsimd's `main` (executor/op-cuda/src/client/main.cpp:23-105).
//   DEEPX_PORT     UDP port (default 9090, op-cuda's port and the front's default endpoint)
//   DEEPX_DEVICE   HIP device ordinal (default 0)
//   DEEPX_BIND     local IPv4 address to bind (default: any, as the reference)
//   DEEPX_REMOTE_QUIT 1: honour the `__quit__` line from any source address (default: loopback only)
//   DEEPX_IR_LOG   1|true: echo every instruction
//   DEEPX_SYNC     1: wait for the device before every reply (default: reply at launch, as op-cuda does)
//   DEEPX_STREAMS  n >= 2: independent kernel-only lines of a datagram go to n side streams in turn and overlap
//   DEEPX_DEFER    1: hold lines that can share a launch with the next one (DEEPX_DEFER_US: longest wait for it, default 200)
//   DEEPX_POOL     0: every tensor's storage comes from and goes back to the driver, as in the reference (default: freed
//                  blocks are kept, up to DXH_POOL_MAX_MB or half the device's memory, and handed out again)
//   DEEPX_ZERO_AT_ALLOC 1: `newtensor` launches its zero fill at once (default: the first launch that names the tensor makes
//                  the fill, or drops it when it overwrites the whole tensor)
//   DEEPX_OPLIST   path: write the generated op table (markdown) there, as the reference writes
//                  docs/executor/op-mem-*/list.md at start-up
#include <csignal>
#include <cstdlib>
#include <fstream>
#include <iostream>
#include "udpserver.hpp"

static deepx::UdpServer *g_server = nullptr;
static void on_signal(int) { if (g_server) g_server->stop(); }

int main() {
    const char *port_env = std::getenv("DEEPX_PORT");
    const int port = port_env ? std::atoi(port_env) : 9090;
    const char *dev_env = std::getenv("DEEPX_DEVICE");
    int count = 0;
    int rc = dxh_device_count(&count);
    if (rc != DXH_OK || count == 0) {
        std::cerr << "deepx-executor-hip: no HIP device (" << dxh_error_string(rc) << "); tensor ops will answer with errors" << std::endl;
    } else {
        rc = dxh_set_device(dev_env ? std::atoi(dev_env) : 0);
        if (rc != DXH_OK) { std::cerr << "dxh_set_device: " << dxh_error_string(rc) << std::endl; return 1; }
        char name[256];
        if (dxh_device_name(name, sizeof name) == DXH_OK) std::cerr << "deepx-executor-hip: " << name << std::endl;
    }
    deepx::Executor ex;
    if (const char *oplist = std::getenv("DEEPX_OPLIST")) {
        std::ofstream md(oplist);
        if (md.is_open()) md << ex.factory.print_markdown("op-mem-hip");
    }
    deepx::UdpServer server(port);
    if (!server.open()) return 1;
    g_server = &server;
    std::signal(SIGINT, on_signal);
    std::signal(SIGTERM, on_signal);
    std::cerr << "deepx-executor-hip: listening on udp " << port << std::endl;
    server.serve(ex);
    return 0;
}
