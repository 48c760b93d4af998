// ir.hpp — the deepxIR text protocol: one instruction per line in, one status line out.
//
//   request : name(<param>, ...)->(<param>, ...) // key=value key=value ...
//   param   : [category[<precision>]:]text          e.g. tensor<float32>:a   vector<int32>:[0 2 1 3]
//   reply   : "<id> ok// recv_at=<ms> start_at=<ms> finish_at=<ms>[ message]"
//
// Grammar and reply format follow executor/deepxcore/src/deepx/tf/tf.cpp:12-43 (Param),
// :74-122 (metadata), :125-192 (name/args/returns split), :299-316 (TF::parse), :327-365
// (to_string) and executor/deepxcore/src/deepx/tf/tf.hpp:183-231 (OpResp); the emitting side is
// front/py/deepx/nn/deepxir.py:133-159.
#pragma once
#include <chrono>
#include <cstdint>
#include <memory>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>
#include "dtype.hpp"

namespace deepx {

class Mem;

inline void trim_spaces(std::string &s) {
    size_t a = s.find_first_not_of(' ');
    if (a == std::string::npos) { s.clear(); return; }
    s = s.substr(a, s.find_last_not_of(' ') - a + 1);
}
inline bool text_is_float(const std::string &s) {
    try { (void)std::stof(s); return true; } catch (...) { return false; }
}
inline bool text_is_int(const std::string &s) {
    try { (void)std::stoi(s); return true; } catch (...) { return false; }
}

struct Param {
    TypeDef dtype;
    std::string textvalue;
    Param() = default;
    Param(const std::string &text, DataCategory c, Precision p) : dtype(c, p), textvalue(text) {}

    // "type:value" split at the FIRST colon; a bare word is both type text and value
    static Param parse(const std::string &raw) {
        Param p;
        size_t colon = raw.find(':');
        if (colon != std::string::npos) {
            std::string type = raw.substr(0, colon), value = raw.substr(colon + 1);
            trim_spaces(type);
            trim_spaces(value);
            if (!type.empty()) { p.dtype = typedef_from(type); p.textvalue = value; return p; }
            p.dtype = typedef_from(value);
            p.textvalue = value;
            return p;
        }
        std::string value = raw;
        trim_spaces(value);
        p.dtype = typedef_from(value);
        p.textvalue = value;
        return p;
    }
    std::string to_string() const { return typedef_str(dtype) + ":" + textvalue; }
};

using TimePoint = std::chrono::system_clock::time_point;
inline int64_t epoch_ms(TimePoint t) {
    return std::chrono::duration_cast<std::chrono::milliseconds>(t.time_since_epoch()).count();
}
// the reference builds time points with system_clock::from_time_t(stod(text)): whole seconds
inline TimePoint from_seconds_text(const std::string &s) {
    return std::chrono::system_clock::from_time_t((std::time_t)std::stod(s));
}

struct TFMetadata {
    std::string author;
    int id = 0;
    TimePoint created_at = TimePoint::min(), sent_at = TimePoint::min(), recv_at = TimePoint::min();
    int benchmark_repeat = 0;

    void parse(const std::string &meta) {
        static const char *blank = " \t\n\r\f\v";  // what `stream >> word` skips; no stream here: this runs for every line
        for (size_t b = 0; (b = meta.find_first_not_of(blank, b)) != std::string::npos;) {
            size_t e = meta.find_first_of(blank, b);
            if (e == std::string::npos) e = meta.size();
            const std::string kv = meta.substr(b, e - b);
            b = e;
            size_t eq = kv.find('=');
            if (eq == std::string::npos) continue;
            std::string k = kv.substr(0, eq), v = kv.substr(eq + 1);
            if (k == "id") id = std::stoi(v);
            else if (k == "author") author = v;
            else if (k == "created_at") created_at = from_seconds_text(v);
            else if (k == "sent_at") sent_at = from_seconds_text(v);
            else if (k == "recv_at") recv_at = from_seconds_text(v);
            else if (k == "benchmark.repeat") benchmark_repeat = std::stoi(v);
        }
    }
    std::string to_string() const {
        std::ostringstream o;
        if (!author.empty()) o << "author=" << author << " ";
        if (id > 0) o << "id=" << id << " ";
        if (created_at != TimePoint::min()) o << "created_at=" << epoch_ms(created_at) << " ";
        if (sent_at != TimePoint::min()) o << "sent_at=" << epoch_ms(sent_at) << " ";
        if (recv_at != TimePoint::min()) o << "recv_at=" << epoch_ms(recv_at) << " ";
        if (benchmark_repeat > 0) o << "benchmark.repeat=" << benchmark_repeat << " ";
        return o.str();
    }
};

inline std::vector<Param> parse_params(const std::string &list) {
    std::vector<Param> out;
    for (size_t b = 0; b <= list.size();) {
        size_t e = list.find(',', b);
        if (e == std::string::npos) e = list.size();
        std::string item = list.substr(b, e - b);
        trim_spaces(item);
        if (!item.empty()) out.push_back(Param::parse(item));
        b = e + 1;
    }
    return out;
}

// TF: one tensor function.  A parsed request is a TF with name/args/returns/metadata; a
// registered implementation is a subclass that overrides run().
class TF {
public:
    std::string name, tftype;
    std::vector<Param> args, returns;
    TFMetadata metadata;
    // true for ops that only launch kernels on Mem's stream (no allocation, host copy, file I/O or
    // fresh random seed): those may be recorded into a HIP graph by the batch path
    bool graph_safe = false;
    // true for ops that write every element of each tensor they return, whatever it held: the zero fill that a fresh
    // tensor still owes (Tensor::zero_pending) is dropped for their results instead of being made
    bool overwrites_results = false;
    // float elementwise ops that dxh_chain can run as part of one launch: its op code, and where the
    // operands sit (1: args 0 and 1 are tensors, 2: tensor then scalar, 3: scalar then tensor, 4: one tensor)
    int chain_code = -1, chain_kind = 0;

    TF() = default;
    explicit TF(const std::string &text) { parse(text); }
    virtual ~TF() = default;

    virtual int run(Mem &mem, std::string &error) { error = "not implemented: " + name; return 1; }
    virtual std::string math_formula() const { return ""; }
    virtual std::shared_ptr<TF> clone() const { return std::make_shared<TF>(*this); }

    void parse(const std::string &input) {
        size_t slashes = input.find("//");
        std::string body = input.substr(0, slashes);
        std::string meta = slashes == std::string::npos ? "" : input.substr(slashes + 2);
        size_t arrow = body.find("->");
        if (arrow == std::string::npos) throw std::runtime_error("Invalid IR format: missing arrow");
        std::string in_part = body.substr(0, arrow), out_part = body.substr(arrow + 2);
        // name ends at the first '(' unless a space comes earlier
        size_t sp = in_part.find(' '), par = in_part.find('(');
        size_t end = (par != std::string::npos && (sp == std::string::npos || par < sp))
                         ? par : (sp != std::string::npos ? sp : in_part.size());
        name = in_part.substr(0, end);
        in_part = in_part.substr(end);
        auto strip = [](std::string s, bool drop_lead_space) {
            size_t l = s.find('('), r = s.rfind(')');
            if (l != std::string::npos && r != std::string::npos) return s.substr(l + 1, r - l - 1);
            if (drop_lead_space && !s.empty() && s[0] == ' ') return s.substr(1);
            return s;
        };
        args = parse_params(strip(in_part, true));
        returns = parse_params(strip(out_part, false));
        metadata.parse(meta);
    }
    std::string to_string(bool show_extra = false) const {
        std::ostringstream o;
        o << name << "(";
        for (size_t i = 0; i < args.size(); ++i) o << (i ? ", " : "") << args[i].to_string();
        o << ")->(";
        for (size_t i = 0; i < returns.size(); ++i) o << (i ? ", " : "") << returns[i].to_string();
        o << ")";
        if (show_extra) o << " //" << metadata.to_string();
        return o.str();
    }
};

struct OpResp {
    int id = 0;
    std::string result, message;
    TimePoint recv_at{}, start_at{}, finish_at{};
    void finish(const std::string &msg) { result = "ok"; finish_at = std::chrono::system_clock::now(); message = msg; }
    void error(const std::string &msg) { result = "error"; finish_at = std::chrono::system_clock::now(); message = msg; }
    // no space between the result word and "//", as tf.hpp:198-213 prints it; the front splits on "//"
    std::string to_string() const {
        std::string o;  // appended by hand: a stream costs more than the rest of a reply
        o.reserve(96 + message.size());
        o += std::to_string(id);
        o += ' ';
        o += result;
        o += "// recv_at=";
        o += std::to_string(epoch_ms(recv_at));
        o += " start_at=";
        o += std::to_string(epoch_ms(start_at));
        o += " finish_at=";
        o += std::to_string(epoch_ms(finish_at));
        if (!message.empty()) { o += ' '; o += message; }
        return o;
    }
};

}  // namespace deepx
