// resp.hpp — the same key-value operations against a Redis server: a minimal RESP2 client over one
// TCP connection (request = array of bulk strings; replies: simple string, error, integer, bulk
// string, array).  It stands where the reference expects redis++ / hiredis
// (executor/heapmem-cuda/README.md:112-114), neither of which is needed for seven commands.
#pragma once
#include <arpa/inet.h>
#include <netdb.h>
#include <sys/socket.h>
#include <unistd.h>
#include <stdexcept>
#include <string>
#include <vector>
#include "kv.hpp"

namespace deepx::heapmem {

struct RespValue {
    char type = '_';  // '+' simple string, '-' error, ':' integer, '$' bulk string, '*' array, '_' nil
    std::string text;
    long long integer = 0;
    std::vector<RespValue> items;
};

class RespKV : public KV {
public:
    RespKV(const std::string &host, int port) {
        addrinfo hints{}, *res = nullptr;
        hints.ai_family = AF_INET;
        hints.ai_socktype = SOCK_STREAM;
        if (getaddrinfo(host.c_str(), std::to_string(port).c_str(), &hints, &res) != 0 || !res)
            throw std::runtime_error("redis: cannot resolve " + host);
        fd_ = ::socket(res->ai_family, res->ai_socktype, res->ai_protocol);
        if (fd_ < 0 || ::connect(fd_, res->ai_addr, res->ai_addrlen) != 0) {
            freeaddrinfo(res);
            if (fd_ >= 0) ::close(fd_);
            throw std::runtime_error("redis: cannot connect to " + host + ":" + std::to_string(port));
        }
        freeaddrinfo(res);
    }
    ~RespKV() override { if (fd_ >= 0) ::close(fd_); }

    RespValue command(const std::vector<std::string> &args) {
        std::string req = "*" + std::to_string(args.size()) + "\r\n";
        for (const auto &a : args) req += "$" + std::to_string(a.size()) + "\r\n" + a + "\r\n";
        size_t sent = 0;
        while (sent < req.size()) {
            ssize_t n = ::send(fd_, req.data() + sent, req.size() - sent, 0);
            if (n <= 0) throw std::runtime_error("redis: send failed");
            sent += (size_t)n;
        }
        RespValue v = read_value();
        if (v.type == '-') throw std::runtime_error("redis: " + v.text);
        return v;
    }

    Hash hgetall(const std::string &key) override {
        RespValue v = command({"HGETALL", key});
        Hash h;
        for (size_t i = 0; i + 1 < v.items.size(); i += 2) h[v.items[i].text] = v.items[i + 1].text;
        return h;
    }
    void hset(const std::string &key, const Hash &fields) override {
        std::vector<std::string> args{"HSET", key};
        for (const auto &kv : fields) { args.push_back(kv.first); args.push_back(kv.second); }
        if (args.size() > 2) command(args);
    }
    long long hincrby(const std::string &key, const std::string &field, long long by) override {
        return command({"HINCRBY", key, field, std::to_string(by)}).integer;
    }
    long long del(const std::string &key) override { return command({"DEL", key}).integer; }
    std::vector<std::string> keys(const std::string &prefix) override {
        RespValue v = command({"KEYS", prefix + "*"});
        std::vector<std::string> out;
        for (const auto &it : v.items) out.push_back(it.text);
        return out;
    }
    void lpush(const std::string &list, const std::string &value) override { command({"LPUSH", list, value}); }
    bool brpop(const std::string &list, int timeout_seconds, std::string &value) override {
        RespValue v = command({"BRPOP", list, std::to_string(timeout_seconds)});
        if (v.type != '*' || v.items.size() != 2) return false;  // nil array on timeout
        value = v.items[1].text;
        return true;
    }

private:
    char read_byte() {
        if (pos_ == len_) {
            ssize_t n = ::recv(fd_, buf_, sizeof buf_, 0);
            if (n <= 0) throw std::runtime_error("redis: connection closed");
            len_ = (size_t)n;
            pos_ = 0;
        }
        return buf_[pos_++];
    }
    std::string read_line() {
        std::string line;
        for (;;) {
            char c = read_byte();
            if (c == '\r') { read_byte(); return line; }
            line += c;
        }
    }
    RespValue read_value() {
        RespValue v;
        v.type = read_byte();
        std::string line = read_line();
        switch (v.type) {
        case '+': case '-': v.text = line; break;
        case ':': v.integer = std::stoll(line); break;
        case '$': {
            long long n = std::stoll(line);
            if (n < 0) { v.type = '_'; break; }
            v.text.reserve((size_t)n);
            for (long long i = 0; i < n; ++i) v.text += read_byte();
            read_byte(); read_byte();
            break;
        }
        case '*': {
            long long n = std::stoll(line);
            if (n < 0) { v.type = '_'; break; }
            for (long long i = 0; i < n; ++i) v.items.push_back(read_value());
            break;
        }
        default: throw std::runtime_error("redis: unexpected reply type");
        }
        return v;
    }

    int fd_ = -1;
    char buf_[4096];
    size_t pos_ = 0, len_ = 0;
};

}  // namespace deepx::heapmem
