// executor.hpp — one deepxIR line in, one reply line out.
//
// This is the body of the reference's main loop (executor/op-ompsimd/src/client/main.cpp:48-101,
// executor/op-cuda/src/client/main.cpp) without the socket: parse, look the op up, run it
// (benchmark.repeat times when asked), stamp recv/start/finish, answer "ok" or "error".
// Unlike the reference nothing here can take the process down: malformed IR, unknown ops,
// missing tensors, shape errors and HIP errors all become "error" replies.
#pragma once
#include <cstdlib>
#include <cstring>
#include <iostream>
#include <mutex>
#include <string>
#include "factory.hpp"
#include "mem.hpp"

namespace deepx {

class Executor {
public:
    Mem mem;
    TfFactory factory;
    bool ir_log = false;    // DEEPX_IR_LOG=1|true echoes every instruction (main.cpp:17-21)
    bool sync_each = true;  // wait for the kernels before stamping finish_at; DEEPX_SYNC=0 replies at launch like op-cuda
    bool has_device = false;

    Executor() {
        register_all(factory);
        const char *e = std::getenv("DEEPX_IR_LOG");
        ir_log = e && (!std::strcmp(e, "1") || !strcasecmp(e, "true"));
        const char *s = std::getenv("DEEPX_SYNC");
        if (s && !std::strcmp(s, "0")) sync_each = false;
        int count = 0;
        has_device = dxh_device_count(&count) == DXH_OK && count > 0;
    }

    std::string execute(const std::string &line, TimePoint recv_at = std::chrono::system_clock::now()) {
        std::lock_guard<std::mutex> lock(mu_);
        OpResp resp;
        resp.recv_at = recv_at;
        resp.start_at = recv_at;
        TF call;
        try {
            call.parse(line);
        } catch (const std::exception &e) {
            resp.error(e.what());
            return resp.to_string();
        }
        call.metadata.recv_at = recv_at;
        resp.id = call.metadata.id;
        if (ir_log) std::cout << "~" << call.to_string(true) << std::endl;
        std::string why;
        auto tf = factory.get_tf(call, &why);
        if (!tf) {
            std::cerr << why << std::endl;
            resp.error("op" + call.name + " not found");
            return resp.to_string();
        }
        tf->name = call.name;
        tf->args = call.args;
        tf->returns = call.returns;
        resp.start_at = std::chrono::system_clock::now();
        int rc = 0;
        std::string message;
        const int repeat = tf->metadata.benchmark_repeat > 1 ? tf->metadata.benchmark_repeat : 1;
        for (int i = 0; i < repeat && rc == 0; ++i) rc = tf->run(mem, message);
        if (rc == 0 && sync_each && has_device) {
            int s = dxh_stream_sync(nullptr);
            if (s != DXH_OK) { rc = 1; message = std::string("hip: ") + dxh_error_string(s); }
        }
        if (rc != 0) {
            std::cerr << message << std::endl;
            resp.error(message);
        } else {
            resp.finish("");
        }
        return resp.to_string();
    }

private:
    std::mutex mu_;
};

}  // namespace deepx
