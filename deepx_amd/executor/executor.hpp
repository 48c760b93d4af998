// executor.hpp — one deepxIR line in, one reply line out.
//
// This is the body of the reference's main loop (executor/op-ompsimd/src/client/main.cpp:48-101,
// executor/op-cuda/src/client/main.cpp) without the socket: parse, look the op up, run it
// (benchmark.repeat times when asked), stamp recv/start/finish, answer "ok" or "error".
// Unlike the reference nothing here can take the process down: malformed IR, unknown ops,
// missing tensors, shape errors and HIP errors all become "error" replies.
#pragma once
#include <algorithm>
#include <cstdlib>
#include <cstring>
#include <functional>
#include <iostream>
#include <mutex>
#include <sstream>
#include <string>
#include <unordered_map>
#include <unordered_set>
#include <vector>
#include "factory.hpp"
#include "mem.hpp"
#include "stream_picker.hpp"

namespace deepx {

class Executor {
public:
    Mem mem;
    TfFactory factory;
    bool ir_log = false;    // DEEPX_IR_LOG=1|true echoes every instruction (main.cpp:17-21)
    // Replies go out when the kernels of a line have been launched, as op-cuda's do (its main loop
    // never waits for the device, executor/op-cuda/src/client/main.cpp:60-104): kernels of later
    // lines queue up behind them on the same stream, and every op that hands data to the host
    // (save, print) waits for the device itself.  One launch-and-wait round trip costs 11.5 us on
    // this runtime whatever the kernel, 250 us of a 22-line block.  DEEPX_SYNC=1 waits for the
    // device before every reply (finish_at is then the end of the kernels, as on op-ompsimd).
    bool sync_each = false;
    bool has_device = false;
    // DEEPX_GRAPH=1: a datagram of several graph-safe lines that arrives a second time is recorded
    // into a HIP graph and replayed from then on (one launch instead of one per kernel)
    bool use_graphs = false;
    // Inside a batch, consecutive float elementwise lines over tensors of one dtype and size run as
    // one launch (dxh_chain): same bits in every output, operands that the run itself produced are
    // not read back from memory.  DEEPX_FUSE=0 turns it off.
    bool use_fusion = true;
    // DEEPX_DEFER=1: the front sends one line per datagram and waits for the reply before it sends the next
    // (front/py/deepx/scheduler/client/udpconn.py:17-48), so on its own it never hands over two lines that
    // could share a launch.  With this switch a line that can start or extend a run (a float elementwise line
    // and its kin, a matmul on the left operand of the one before) is answered at once and HELD; the run goes
    // out — as one launch where the library takes it, as separate ones otherwise — when a line arrives that
    // does not extend it, when flush() is called, or when the server has seen no datagram for a moment.  A
    // line is held only after it has been checked against the tensor store like a line of a batch (operands
    // exist, dtypes and extents agree), and nothing else executes while lines are held, so the tensors end up
    // as line-by-line execution leaves them; the reply of a held line carries the time it was accepted.
    // Off with DEEPX_SYNC=1 (a reply then promises finished kernels) and with DEEPX_FUSE=0.
    bool defer = false;
    // DEEPX_STREAMS=n (n >= 2): kernel-only lines (of a batch, or sent one by one) are spread over n side streams so that launches which
    // do not depend on each other overlap (the end of one runs under the start of the next; ten reductions over one
    // [8192,8192] tensor: 341 -> 313 us); a line that reads or writes what a launch in flight wrote, or writes what one
    // reads, goes behind that launch on its stream (see pick_stream).  The tensors end up as in-order execution leaves
    // them.  Each side stream has a scratch buffer of its own.  Off (1) by default.
    int streams = 1;
    struct Stats { uint64_t batches = 0, graph_captures = 0, graph_replays = 0, graph_rejects = 0, fused_runs = 0, fused_lines = 0, matmul_groups = 0, matmul_lines = 0, held_lines = 0, flushes = 0, side_launches = 0; } stats;
    // Where the host time of a line goes (steady clock, nanoseconds summed over `lines` calls of
    // execute()): parsing the text, finding and cloning the registered op, its wrapper up to the
    // kernel launch, the wait for the device, formatting the reply.  Off unless DEEPX_PROFILE=1.
    bool profile = false;
    struct Profile { uint64_t lines = 0, parse_ns = 0, match_ns = 0, run_ns = 0, sync_ns = 0, reply_ns = 0; } prof;

    Executor() {
        // the kernel library found at run time must be the one this host code was compiled against
        if (dxh_version() != DXH_ABI_VERSION)
            throw std::runtime_error("libdxhip.so has ABI " + std::to_string(dxh_version()) + ", this executor was built for " + std::to_string(DXH_ABI_VERSION));
        register_all(factory);
        const char *e = std::getenv("DEEPX_IR_LOG");
        ir_log = e && (!std::strcmp(e, "1") || !strcasecmp(e, "true"));
        const char *s = std::getenv("DEEPX_SYNC");
        if (s) sync_each = !std::strcmp(s, "1");
        int count = 0;
        has_device = dxh_device_count(&count) == DXH_OK && count > 0;
        const char *g = std::getenv("DEEPX_GRAPH");
        use_graphs = g && !std::strcmp(g, "1");
        const char *pr = std::getenv("DEEPX_PROFILE");
        profile = pr && !std::strcmp(pr, "1");
        const char *fuse = std::getenv("DEEPX_FUSE");
        if (fuse && !std::strcmp(fuse, "0")) use_fusion = false;
        const char *df = std::getenv("DEEPX_DEFER");
        defer = df && !std::strcmp(df, "1");
        if (const char *ns = std::getenv("DEEPX_STREAMS")) streams = std::max(1, std::min(8, std::atoi(ns)));
    }
    ~Executor() {
        try { flush(); } catch (const std::exception &e) { std::cerr << "held lines lost at shutdown: " << e.what() << std::endl; }
        for (auto &kv : graphs_) drop_graph(kv.second);
        if (graph_event_) dxh_event_destroy(graph_event_);
        if (graph_stream_) dxh_stream_destroy(graph_stream_);
        if (!side_.empty()) dxh_device_sync();
        for (Side &sd : side_) { dxh_event_destroy(sd.event); dxh_stream_destroy(sd.stream); }
    }

    // lines accepted under `defer` and not yet launched
    size_t held() {
        std::lock_guard<std::recursive_mutex> lock(mu_);
        return held_items_.size();
    }
    // launches what is held; failures (none are expected: the lines were checked when they were accepted) go to stderr
    void flush() {
        std::lock_guard<std::recursive_mutex> lock(mu_);
        if (held_items_.empty()) return;
        std::vector<Item> items;
        items.swap(held_items_);
        held_run_.reset();
        ++stats.flushes;
        for (const std::string &reply : run_items(items, "", false, items[0].resp.recv_at))
            if (reply.find(" ok") == std::string::npos) std::cerr << "held line failed: " << reply << std::endl;
    }

    std::string execute(const std::string &line, TimePoint recv_at = std::chrono::system_clock::now()) {
        std::lock_guard<std::recursive_mutex> lock(mu_);
        using Clock = std::chrono::steady_clock;
        Clock::time_point mark = profile ? Clock::now() : Clock::time_point();
        auto lap = [&](uint64_t &slot) {
            if (!profile) return;
            const Clock::time_point now = Clock::now();
            slot += (uint64_t)std::chrono::duration_cast<std::chrono::nanoseconds>(now - mark).count();
            mark = now;
        };
        if (profile) ++prof.lines;
        OpResp resp;
        resp.recv_at = recv_at;
        resp.start_at = recv_at;
        TF call;
        try {
            call.parse(line);
        } catch (const std::exception &e) {
            flush();
            resp.error(e.what());
            return resp.to_string();
        }
        lap(prof.parse_ns);
        call.metadata.recv_at = recv_at;
        resp.id = call.metadata.id;
        if (ir_log) std::cout << "~" << call.to_string(true) << std::endl;
        std::string why;
        auto tf = factory.get_tf(call, &why);
        if (!tf) {
            flush();
            std::cerr << why << std::endl;
            resp.error("op" + call.name + " not found");
            return resp.to_string();
        }
        tf->name = call.name;
        tf->args = call.args;
        tf->returns = call.returns;
        lap(prof.match_ns);
        if (defer && !sync_each && use_fusion && has_device) {
            // hold the line if it extends what is held into one longer run, or — after what is held has gone
            // out — if it can start a run of its own
            bool hold = false;
            if ((tf->chain_kind != 0 || tf->name == "matmul") && tf->metadata.benchmark_repeat <= 1) {
                hold = held_run_.extend(tf.get(), mem);
                if (!hold && held_run_.size() > 0) {
                    flush();  // also forgets the run
                    hold = held_run_.extend(tf.get(), mem);
                }
            }
            if (hold) {
                ++stats.held_lines;
                resp.start_at = std::chrono::system_clock::now();
                resp.finish("");
                held_items_.emplace_back();
                held_items_.back().call = std::move(call);
                held_items_.back().tf = tf;
                held_items_.back().resp = resp;
                if (held_items_.size() >= 64) flush();  // a run that never ends (products on one operand, say) still goes out
                return resp.to_string();
            }
        }
        // An allocation under a name that no held line mentions touches nothing they use (held lines were checked against
        // the tensors that existed when they were accepted), so it need not end their run: the front allocates every
        // result right before the line that computes it (front/py/deepx/nn/functional/reduce.py:19-20,
        // leaffunc.py:30-38), and a run would never grow otherwise.  Under a name they do mention it replaces a tensor
        // they are about to use, and comes after them like any other line.
        bool beside_held = tf->name == "newtensor" && !held_items_.empty() && call.returns.size() == 1;
        for (size_t h = 0; h < held_items_.size() && beside_held; ++h) beside_held = !mentions(held_items_[h].call, call.returns[0].textvalue);
        if (!beside_held)
            flush();  // whatever is held comes first (also when a switch was turned while lines were held)
        resp.start_at = std::chrono::system_clock::now();
        int rc = 0;
        std::string message;
        const int repeat = tf->metadata.benchmark_repeat > 1 ? tf->metadata.benchmark_repeat : 1;
        if (streams >= 2 && has_device) {  // a line on its own may leave the default stream like a line of a batch
            std::vector<Item> one(1);
            one[0].call = call;
            one[0].tf = tf;
            pick_stream(one, {tf}, 0);
        }
        std::vector<std::shared_ptr<Tensor>> dropped;
        settle(*tf, dropped);
        for (int i = 0; i < repeat && rc == 0; ++i) rc = tf->run(mem, message);
        if (rc != 0) make_good(dropped);
        mem.stream = nullptr;
        mem.scratch_of = nullptr;
        lap(prof.run_ns);
        if (rc == 0 && sync_each && has_device) {
            int s = side_.empty() ? dxh_stream_sync(nullptr) : dxh_device_sync();
            if (s != DXH_OK) { rc = 1; message = std::string("hip: ") + dxh_error_string(s); }
        }
        lap(prof.sync_ns);
        if (rc != 0) {
            std::cerr << message << std::endl;
            resp.error(message);
        } else {
            resp.finish("");
        }
        std::string reply = resp.to_string();
        lap(prof.reply_ns);
        return reply;
    }

    // All lines of one datagram (udpserver.cpp:49-58 splits them the same way), one reply per line,
    // in order.  The kernels of the whole datagram are launched back to back and waited for once,
    // instead of once per line; finish_at of every line is then the end of the batch.  Each line
    // still succeeds or fails on its own, as when sent one by one.
    std::vector<std::string> execute_batch(const std::vector<std::string> &lines, TimePoint recv_at = std::chrono::system_clock::now()) {
        if (lines.size() == 1) return {execute(lines[0], recv_at)};
        std::lock_guard<std::recursive_mutex> lock(mu_);
        flush();  // lines held from earlier datagrams come first
        ++stats.batches;
        // graphs are keyed by the instruction text without the per-call metadata (ids, timestamps)
        std::string key;
        for (const std::string &line : lines) {
            size_t end = line.find("//");
            if (end == std::string::npos) end = line.size();
            while (end > 0 && line[end - 1] == ' ') --end;
            key.append(line, 0, end);
            key += '\n';
        }
        if (use_graphs && has_device) {  // a batch recorded earlier whose tensors are all where they were: no parsing at all
            auto hit = graphs_.find(key);
            if (hit != graphs_.end() && pins_hold(hit->second)) {
                std::vector<int> ids;
                bool plain = true;  // ids readable, no benchmark.repeat: otherwise take the parsing path
                try {
                    for (const std::string &line : lines) {
                        TFMetadata m;
                        size_t meta = line.find("//");
                        if (meta != std::string::npos) m.parse(line.substr(meta + 2));
                        plain = plain && m.benchmark_repeat <= 1;
                        ids.push_back(m.id);
                    }
                } catch (const std::exception &) {
                    plain = false;
                }
                if (plain && launch_graph(hit->second)) {
                    ++stats.graph_replays;
                    std::vector<std::string> replies;
                    replies.reserve(lines.size());
                    for (int id : ids) {
                        OpResp resp;
                        resp.recv_at = resp.start_at = recv_at;
                        resp.id = id;
                        resp.finish("");
                        replies.push_back(resp.to_string());
                    }
                    return replies;
                }
            }
        }
        std::vector<Item> items(lines.size());
        bool graphable = use_graphs && has_device;
        for (size_t i = 0; i < lines.size(); ++i) {
            Item &it = items[i];
            it.resp.recv_at = it.resp.start_at = recv_at;
            try {
                it.call.parse(lines[i]);
            } catch (const std::exception &e) {
                it.resp.error(e.what());
                it.failed = true;
                graphable = false;
                continue;
            }
            it.call.metadata.recv_at = recv_at;
            it.resp.id = it.call.metadata.id;
            if (ir_log) std::cout << "~" << it.call.to_string(true) << std::endl;
            std::string why;
            it.tf = factory.get_tf(it.call, &why);
            if (!it.tf) {
                std::cerr << why << std::endl;
                it.resp.error("op" + it.call.name + " not found");
                it.failed = true;
                graphable = false;
                continue;
            }
            it.tf->name = it.call.name;
            it.tf->args = it.call.args;
            it.tf->returns = it.call.returns;
            graphable = graphable && it.tf->graph_safe && it.tf->metadata.benchmark_repeat <= 1 && !uses_named_arg(it.call);
        }
        // Allocations first: a `newtensor` line whose tensor no earlier line of the batch names moves to the front (in
        // order among themselves), so that the compute lines it sat between can share a launch.  Replies keep the
        // order of the lines.
        std::vector<size_t> order;
        {
            std::vector<size_t> rest;
            std::unordered_set<std::string> named;  // every word of the lines so far that could be a tensor's name
            for (size_t i = 0; i < items.size(); ++i) {
                const bool hoist = !items[i].failed && items[i].tf && items[i].call.name == "newtensor" && items[i].call.returns.size() == 1 &&
                                   !named.count(items[i].call.returns[0].textvalue);
                (hoist ? order : rest).push_back(i);
                if (items[i].failed) {  // a line that did not parse: anything between its punctuation counts
                    each_word(lines[i], " []()<>,:", [&](const std::string &w) { named.insert(w); });
                } else {
                    for (const std::vector<Param> *ps : {&items[i].call.args, &items[i].call.returns})
                        for (const Param &prm : *ps) each_word(prm.textvalue, " []", [&](const std::string &w) { named.insert(w); });
                }
            }
            if (order.empty() || order.size() == items.size()) order.clear();
            else order.insert(order.end(), rest.begin(), rest.end());
        }
        if (order.empty()) return run_items(items, key, graphable, recv_at);
        std::vector<Item> moved(items.size());
        for (size_t k = 0; k < order.size(); ++k) moved[k] = std::move(items[order[k]]);
        const std::vector<std::string> out = run_items(moved, key, false, recv_at);
        std::vector<std::string> replies(out.size());
        for (size_t k = 0; k < order.size(); ++k) replies[order[k]] = out[k];
        return replies;
    }

private:
    struct Item { TF call; std::shared_ptr<TF> tf; OpResp resp; bool failed = false; };

    // Parsed and matched lines, in order: runs where lines can share a launch, single launches otherwise,
    // as one recorded graph when `graphable`; one reply per line.
    std::vector<std::string> run_items(std::vector<Item> &items, const std::string &key, bool graphable, TimePoint recv_at) {
        std::vector<std::shared_ptr<TF>> tfs(items.size());
        for (size_t i = 0; i < items.size(); ++i) if (!items[i].failed) tfs[i] = items[i].tf;
        // Runs line i, or a run of lines that starts at i as one launch; returns how many lines that were.
        // A run that cannot be launched after all falls back to its first line alone.
        auto run_next = [&](size_t i, std::string &message, int &rc) -> size_t {
            std::vector<std::shared_ptr<Tensor>> dropped;
            if (use_fusion && has_device) {
                const size_t len = chain_length(tfs, i, mem);
                if (len >= 2) {
                    for (size_t j = i; j < i + len; ++j) settle(*tfs[j], dropped);
                    try { rc = run_chain(tfs, i, len, mem, message); } catch (const std::exception &e) { rc = 1; message = e.what(); }
                    if (rc == 0) { ++stats.fused_runs; stats.fused_lines += len; return len; }
                    make_good(dropped);
                    message.clear();
                }
                const size_t group = matmul_group_length(tfs, i, mem);
                if (group >= 2) {
                    for (size_t j = i; j < i + group; ++j) settle(*tfs[j], dropped);
                    try { rc = run_matmul_group(tfs, i, group, mem, message); } catch (const std::exception &e) { rc = 1; message = e.what(); }
                    if (rc == 0) { ++stats.matmul_groups; stats.matmul_lines += group; return group; }
                    make_good(dropped);
                    message.clear();
                }
            }
            const int repeat = items[i].tf->metadata.benchmark_repeat > 1 ? items[i].tf->metadata.benchmark_repeat : 1;
            rc = 0;
            settle(*items[i].tf, dropped);
            for (int r = 0; r < repeat && rc == 0; ++r) rc = items[i].tf->run(mem, message);
            if (rc != 0) make_good(dropped);
            return 1;
        };
        bool done = false;
        if (graphable) {
            auto run_all = [&]() {
                for (size_t i = 0; i < items.size();) {
                    std::string message;
                    int rc = 0;
                    const size_t used = run_next(i, message, rc);
                    if (rc != 0) return false;
                    i += used;
                }
                return true;
            };
            if (run_as_graph(key, items.size(), run_all, [&](size_t i) -> const TF & { return items[i].call; })) {
                for (Item &it : items) { it.resp.start_at = recv_at; it.resp.finish(""); }
                done = true;
            }
        }
        if (!done) {
            for (size_t i = 0; i < items.size();) {
                if (items[i].failed) { ++i; continue; }
                const TimePoint started = std::chrono::system_clock::now();
                int rc = 0;
                std::string message;
                pick_stream(items, tfs, i);
                const size_t used = run_next(i, message, rc);
                mem.stream = nullptr;
                mem.scratch_of = nullptr;
                for (size_t j = i; j < i + used; ++j) items[j].resp.start_at = started;
                if (rc != 0) {
                    std::cerr << message << std::endl;
                    items[i].resp.error(message);
                    items[i].failed = true;
                }
                i += used;
            }
            std::string sync_error;
            if (sync_each && has_device) {
                int s = side_.empty() ? dxh_stream_sync(nullptr) : dxh_device_sync();
                if (s != DXH_OK) sync_error = std::string("hip: ") + dxh_error_string(s);
            }
            for (Item &it : items) {
                if (it.failed) continue;
                if (!sync_error.empty()) it.resp.error(sync_error);
                else it.resp.finish("");
            }
        }
        std::vector<std::string> replies;
        replies.reserve(items.size());
        for (Item &it : items) replies.push_back(it.resp.to_string());
        return replies;
    }

    // Which stream the launch that starts at line i goes to (see `streams`).  The decision is StreamPicker's
    // (stream_picker.hpp): the next side stream in turn for a kernel-only launch that clashes with nothing in flight,
    // the stream it clashes with otherwise — after that stream has been told to wait for events recorded on the other
    // streams it clashes with — and the default stream for anything that is not kernel-only, behind a join of the side
    // streams (join_side_streams).  A launch on the default stream waits for all side streams and makes them wait for it
    // (they are ordinary blocking streams): correct, and slow on this runtime (a launch there between launches on other
    // streams costs about 60 us), which is why clashes do not go there.
    void pick_stream(const std::vector<Item> &items, const std::vector<std::shared_ptr<TF>> &tfs, size_t i) {
        mem.stream = nullptr;
        mem.scratch_of = nullptr;
        if (streams < 2 || !has_device) return;
        size_t len = 1;  // the lines run_next will take, or more: a superset of their tensors is as safe
        if (use_fusion) len = std::max<size_t>({len, chain_length(tfs, i, mem), matmul_group_length(tfs, i, mem)});
        std::vector<std::string> reads, writes;
        bool kernel_only = true;
        for (size_t j = i; j < i + len && j < items.size(); ++j) {
            if (items[j].failed || !items[j].tf) { kernel_only = false; break; }
            kernel_only = kernel_only && items[j].tf->graph_safe && items[j].tf->metadata.benchmark_repeat <= 1;
            names_in(items[j].call.args, reads);
            names_in(items[j].call.returns, writes);
            each_tensor(items[j].call.args, [&](const std::shared_ptr<Tensor> &t) {  // an argument that is still owed its zero fill is written first
                if (t->zero_pending) names_in(items[j].call.args, writes);
            });
        }
        while (side_.size() < (size_t)streams) {
            Side sd;
            if (dxh_stream_create(&sd.stream) != DXH_OK || !sd.stream) { streams = 1; picker_.resize(0); return; }
            if (dxh_event_create(&sd.event) != DXH_OK || !sd.event) { dxh_stream_destroy(sd.stream); streams = 1; picker_.resize(0); return; }
            side_.push_back(sd);
        }
        if (picker_.streams() != (int)side_.size()) picker_.resize((int)side_.size());
        const std::vector<int> busy = picker_.busy();
        const bool flying = graph_flying_;
        const StreamPicker::Choice c = picker_.place(reads, writes, kernel_only, flying);
        graph_flying_ = false;
        if (c.stream < 0) {  // the default stream
            join_side_streams(busy, flying);
            return;
        }
        for (int other : c.wait_for) {
            if (dxh_event_record(side_[(size_t)other].event, side_[(size_t)other].stream) != DXH_OK ||
                dxh_stream_wait_event(side_[(size_t)c.stream].stream, side_[(size_t)other].event) != DXH_OK) {
                picker_.abandon();
                return;  // could not order them: the default stream does
            }
        }
        mem.stream = mem.scratch_of = side_[(size_t)c.stream].stream;
        ++stats.side_launches;
    }
    // `fn(word)` for every run of characters of `text` that holds none of `separators`
    template <typename Fn>
    static void each_word(const std::string &text, const char *separators, Fn fn) {
        for (size_t b = 0; b < text.size();) {
            b = text.find_first_not_of(separators, b);
            if (b == std::string::npos) break;
            size_t e = text.find_first_of(separators, b);
            if (e == std::string::npos) e = text.size();
            fn(text.substr(b, e - b));
            b = e;
        }
    }
    // `fn(tensor)` for every existing tensor among the words of `ps` (bare names, typed params and [a b c] lists alike)
    template <typename Fn>
    void each_tensor(const std::vector<Param> &ps, Fn fn) const {
        for (const Param &p : ps)
            each_word(p.textvalue, " []", [&](const std::string &w) { if (auto found = mem.findtensor(w)) fn(found); });
    }
    // A tensor fresh from `newtensor` reads as zeros but may not hold them yet (Tensor::zero_pending).  Before anything is
    // launched for `tf`: every such tensor among its arguments is filled now, on the stream the launch goes to, and so is
    // one among its results — unless the op writes every element of its results anyway: then the fill is dropped, and
    // `dropped` keeps the tensor so that a launch that fails after all can make it (make_good).  `deltensor` settles
    // nothing: nobody will read what it names.
    void settle(const TF &tf, std::vector<std::shared_ptr<Tensor>> &dropped) {
        if (tf.name == "deltensor") return;
        each_tensor(tf.args, [&](const std::shared_ptr<Tensor> &t) {
            if (t->zero_pending) t->fill_zero(mem.stream);
        });
        each_tensor(tf.returns, [&](const std::shared_ptr<Tensor> &t) {
            if (!t->zero_pending) return;
            if (tf.overwrites_results && !mem.recording) { t->zero_pending = false; dropped.push_back(t); }
            else t->fill_zero(mem.stream);
        });
    }
    void make_good(std::vector<std::shared_ptr<Tensor>> &dropped) {
        for (auto &t : dropped) t->fill_zero(mem.stream);
        dropped.clear();
    }
    // Orders everything the `busy` side streams have been given so far before whatever any stream is given from now on.
    // A launch on the default stream would do that by itself (it waits for every blocking stream, and they for it), but a
    // line sent there need not launch anything: `deltensor`, `renametensor` and `argset` are host work, an empty tensor
    // has no kernel, a line can fail before its launch — and the picker has forgotten what was in flight either way.  So
    // the join is made of events: each busy stream records one, and the default stream and every other side stream wait for it.
    // A replayed graph that may still be running on its own stream (`graph_too`) is waited for the same way.
    void join_side_streams(const std::vector<int> &busy, bool graph_too) {
        bool ok = true;
        if (graph_too && graph_stream_) {
            if (!graph_event_ && dxh_event_create(&graph_event_) != DXH_OK) graph_event_ = nullptr;
            ok = graph_event_ && dxh_event_record(graph_event_, graph_stream_) == DXH_OK && dxh_stream_wait_event(nullptr, graph_event_) == DXH_OK;
            for (size_t b = 0; b < side_.size() && ok; ++b) ok = dxh_stream_wait_event(side_[b].stream, graph_event_) == DXH_OK;
        }
        for (int a : busy) {
            ok = ok && dxh_event_record(side_[(size_t)a].event, side_[(size_t)a].stream) == DXH_OK &&
                 dxh_stream_wait_event(nullptr, side_[(size_t)a].event) == DXH_OK;
            for (size_t b = 0; b < side_.size() && ok; ++b)
                if ((int)b != a) ok = dxh_stream_wait_event(side_[b].stream, side_[(size_t)a].event) == DXH_OK;
        }
        if (!ok) dxh_device_sync();  // the one join that needs no event
    }
    // does a call name `word` among its arguments or results (bare, typed, or inside a [a b c] list)
    static bool mentions(const TF &call, const std::string &word) {
        bool found = false;
        for (const std::vector<Param> *ps : {&call.args, &call.returns})
            for (const Param &p : *ps) each_word(p.textvalue, " []", [&](const std::string &w) { found = found || w == word; });
        return found;
    }
    void names_in(const std::vector<Param> &ps, std::vector<std::string> &names) const {
        for (const Param &p : ps) each_word(p.textvalue, " []", [&](const std::string &w) { if (mem.existstensor(w)) names.push_back(w); });
    }

    // What a recorded graph froze about a tensor: the kernels' pointer arguments and every launch
    // shape derived from its dims (an in-place reshape keeps address and size but not those).
    struct Pinned {
        std::string name; const void *data; int64_t bytes; int dtype; std::vector<int> dims;
        bool same(const void *d, int64_t b, int t, const std::vector<int> &s) const { return data == d && bytes == b && dtype == t && dims == s; }
    };
    struct Graph { void *exec = nullptr; std::vector<Pinned> tensors; const void *workspace = nullptr; };

    // every tensor a call names (bare names, typed params and [a b c] lists alike)
    void tensors_of(const TF &call, std::vector<std::string> &names) const {
        names_in(call.args, names);
        names_in(call.returns, names);
    }
    // a scalar or vector taken from the arg store would be frozen into a recorded graph
    bool uses_named_arg(const TF &call) const {
        bool named = false;
        for (const Param &p : call.args) each_word(p.textvalue, " []", [&](const std::string &w) { named = named || (!mem.existstensor(w) && mem.existarg(w)); });
        return named;
    }
    bool snapshot(size_t n, const std::function<const TF &(size_t)> &call_at, Graph &g) const {
        std::vector<std::string> names;
        for (size_t i = 0; i < n; ++i) tensors_of(call_at(i), names);
        g.tensors.clear();
        for (const std::string &name : names) {
            auto t = mem.gettensor(name);
            g.tensors.push_back({name, t->data, t->shape.bytes(), t->dtype(), t->shape.shape});
        }
        g.workspace = mem.workspace_ptr();
        return true;
    }
    bool pins_hold(const Graph &g) const {
        if (g.workspace != mem.workspace_ptr()) return false;
        for (const Pinned &p : g.tensors) {
            auto t = mem.findtensor(p.name);
            if (!t || !p.same(t->data, t->shape.bytes(), t->dtype(), t->shape.shape)) return false;
        }
        return true;
    }
    // a replay may still be running when replies are sent at launch: wait before its graph goes away
    void drop_graph(Graph &g) {
        if (graph_stream_) dxh_stream_sync(graph_stream_);
        dxh_graph_destroy(g.exec);
        g.exec = nullptr;
    }
    // A recorded graph must not hold the zero fill that a fresh tensor is owed (every replay would clear the tensor again),
    // and a replay reads its tensors as they are: whatever the batch names gets its fill now, on the default stream, which
    // the graph's stream waits for.
    void settle_pins(const Graph &g) {
        for (const Pinned &p : g.tensors) {
            auto t = mem.findtensor(p.name);
            if (t && t->zero_pending) t->fill_zero(nullptr);
        }
    }
    bool launch_graph(const Graph &g) {
        settle_pins(g);
        graph_flying_ = true;
        return dxh_graph_launch(g.exec, graph_stream_) == DXH_OK && (!sync_each || dxh_stream_sync(graph_stream_) == DXH_OK);
    }
    static bool same_pins(const Graph &a, const Graph &b) {
        if (a.workspace != b.workspace || a.tensors.size() != b.tensors.size()) return false;
        for (size_t i = 0; i < a.tensors.size(); ++i)
            if (a.tensors[i].name != b.tensors[i].name ||
                !a.tensors[i].same(b.tensors[i].data, b.tensors[i].bytes, b.tensors[i].dtype, b.tensors[i].dims)) return false;
        return true;
    }

    // Returns true when the whole batch ran (was replayed or recorded and launched) as one graph.
    // false = nothing ran on the device: the caller executes the lines eagerly.  A batch is only
    // recorded on its second arrival (the first, eager, pass also sizes the reduction / matmul
    // workspace), and replayed only while every tensor it names still has the address, size, dtype
    // and dims it was recorded with.
    bool run_as_graph(const std::string &key, size_t n, const std::function<bool()> &run_all,
                      const std::function<const TF &(size_t)> &call_at) {
        if (rejected_.count(key)) return false;
        Graph now;
        try {
            snapshot(n, call_at, now);
        } catch (const std::exception &) {
            return false;  // a missing tensor: the eager path reports it per line
        }
        auto it = graphs_.find(key);
        if (it != graphs_.end() && !same_pins(it->second, now)) {
            drop_graph(it->second);
            graphs_.erase(it);
            it = graphs_.end();
        }
        if (it == graphs_.end()) {
            // bounded memory in a long-lived server: forgetting a text only costs one more eager pass
            if (seen_.size() >= kMaxRemembered) seen_.clear();
            if (rejected_.size() >= kMaxRemembered) rejected_.clear();
            if (seen_.insert(key).second) return false;  // first arrival: run eagerly
            if (!graph_stream_ && dxh_stream_create(&graph_stream_) != DXH_OK) { graph_stream_ = nullptr; return false; }
            settle_pins(now);
            if (dxh_stream_sync(nullptr) != DXH_OK) return false;
            if (dxh_graph_begin_capture(graph_stream_) != DXH_OK) return false;
            mem.stream = graph_stream_;
            mem.recording = true;
            const bool ok = run_all();
            mem.stream = nullptr;
            mem.recording = false;
            void *exec = nullptr;
            int rc = dxh_graph_end_capture(graph_stream_, &exec);
            if (!ok || rc != DXH_OK || !exec) {
                if (exec) dxh_graph_destroy(exec);
                rejected_.insert(key);
                ++stats.graph_rejects;
                return false;
            }
            if (graphs_.size() >= 64) {  // bounded cache: start over rather than track recency
                for (auto &kv : graphs_) drop_graph(kv.second);
                graphs_.clear();
            }
            now.exec = exec;
            it = graphs_.emplace(key, now).first;
            ++stats.graph_captures;
        } else {
            ++stats.graph_replays;
        }
        settle_pins(it->second);
        graph_flying_ = true;
        if (dxh_graph_launch(it->second.exec, graph_stream_) != DXH_OK || (sync_each && dxh_stream_sync(graph_stream_) != DXH_OK)) {
            drop_graph(it->second);
            graphs_.erase(it);
            rejected_.insert(key);
            return false;
        }
        return true;
    }

    std::recursive_mutex mu_;  // flush() is called from inside execute() and execute_batch()
    std::vector<Item> held_items_;
    struct Side { void *stream = nullptr, *event = nullptr; };
    std::vector<Side> side_;  // side streams, created on first use
    StreamPicker picker_;
    bool graph_flying_ = false;
    HeldRun held_run_;  // what the held lines form, kept up to date as they arrive
    void *graph_stream_ = nullptr, *graph_event_ = nullptr;
    std::unordered_map<std::string, Graph> graphs_;
    static constexpr size_t kMaxRemembered = 1024;
    std::unordered_set<std::string> seen_, rejected_;
};

}  // namespace deepx
