// udpserver.hpp — the wire: UDP/IPv4, newline-separated IR lines in, one reply datagram per line.
//
// Protocol of executor/deepxcore/src/client/udpserver.cpp:20-65 (bind INADDR_ANY:<port>, split the
// datagram on '\n', reply to the sender with sendto).  Differences, all to remove crashes: the
// receive buffer is 64 KiB with the terminator inside it (the reference writes buffer[1024]), a
// parse failure answers with an error line instead of unwinding the receiver thread, and replies go
// to the address each datagram came from rather than to "the last client".  One line of its own,
// `__quit__`, ends serve() (the test harness stops the process with it); it is honoured only in a
// datagram whose source address is loopback, unless DEEPX_REMOTE_QUIT=1.  DEEPX_BIND names the local
// address to bind instead of INADDR_ANY (e.g. 127.0.0.1 when the front runs on the same host).
// While the executor holds lines back (DEEPX_DEFER=1) the loop waits at most DEEPX_DEFER_US microseconds
// (default 200) for the next datagram before it launches them, so a pause of the sender never leaves work unlaunched.
#pragma once
#include <arpa/inet.h>
#include <poll.h>
#include <sys/socket.h>
#include <unistd.h>
#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <sstream>
#include <string>
#include "executor.hpp"

namespace deepx {

class UdpServer {
public:
    explicit UdpServer(int port) : port_(port) {}
    ~UdpServer() { if (fd_ >= 0) ::close(fd_); }

    bool open() {
        fd_ = ::socket(AF_INET, SOCK_DGRAM, 0);
        if (fd_ < 0) { perror("socket creation failed"); return false; }
        int rcv = 4 << 20;
        ::setsockopt(fd_, SOL_SOCKET, SO_RCVBUF, &rcv, sizeof rcv);
        sockaddr_in addr{};
        addr.sin_family = AF_INET;
        addr.sin_addr.s_addr = INADDR_ANY;
        if (const char *bind_to = std::getenv("DEEPX_BIND")) {
            if (::inet_pton(AF_INET, bind_to, &addr.sin_addr) != 1) { fprintf(stderr, "DEEPX_BIND: not an IPv4 address: %s\n", bind_to); return false; }
        }
        if (const char *us = std::getenv("DEEPX_DEFER_US")) defer_us_ = std::max(0, std::atoi(us));
        const char *rq = std::getenv("DEEPX_REMOTE_QUIT");
        remote_quit_ = rq && std::string(rq) == "1";
        addr.sin_port = htons((uint16_t)port_);
        if (::bind(fd_, (const sockaddr *)&addr, sizeof addr) < 0) { perror("bind failed"); return false; }
        timeval tv{0, 200000};  // wake up to notice stop()
        ::setsockopt(fd_, SOL_SOCKET, SO_RCVTIMEO, &tv, sizeof tv);
        return true;
    }

    // Receive, execute, reply, until stop().  The front keeps exactly one instruction in flight
    // (front/py/deepx/scheduler/client/udpconn.py:17-48), so executing on the receiving thread
    // serialises ops exactly as the reference's queue + single consumer does.
    void serve(Executor &ex) {
        std::vector<char> buf(65536);
        while (!stop_) {
            if (ex.held() > 0) {  // nothing more within the grace period: launch what is held
                pollfd pfd{fd_, POLLIN, 0};
                timespec grace{defer_us_ / 1000000, (long)(defer_us_ % 1000000) * 1000};
                if (::ppoll(&pfd, 1, &grace, nullptr) <= 0) { ex.flush(); continue; }
            }
            sockaddr_in cli{};
            socklen_t len = sizeof cli;
            ssize_t n = ::recvfrom(fd_, buf.data(), buf.size() - 1, 0, (sockaddr *)&cli, &len);
            if (n <= 0) continue;
            buf[(size_t)n] = '\0';
            TimePoint recv_at = std::chrono::system_clock::now();
            std::istringstream lines(std::string(buf.data(), (size_t)n));
            std::string line;
            std::vector<std::string> batch;
            while (std::getline(lines, line)) {
                if (!line.empty() && line.back() == '\r') line.pop_back();
                if (line.empty()) continue;
                if (line == "__quit__") {
                    const bool loopback = (ntohl(cli.sin_addr.s_addr) >> 24) == 127;
                    if (loopback || remote_quit_) { stop_ = true; break; }
                    continue;  // from elsewhere: neither a command nor an instruction
                }
                batch.push_back(line);
            }
            if (batch.empty()) continue;
            // the lines of one datagram run as one batch: one wait for the device, one reply per line
            for (const std::string &reply : ex.execute_batch(batch, recv_at))
                ::sendto(fd_, reply.data(), reply.size(), 0, (const sockaddr *)&cli, len);
        }
    }
    void stop() { stop_ = true; }

private:
    int port_;
    int fd_ = -1;
    bool remote_quit_ = false;
    int defer_us_ = 200;
    std::atomic<bool> stop_{false};
};

}  // namespace deepx
