// capi.cpp — libdxexec.so: the executor's dispatch core behind a C ABI, so a harness (or an
// embedding scheduler) can feed deepxIR lines without a socket.  Same code path as the UDP binary.
#include <cstring>
#include <sstream>
#include <string>
#include <vector>
#include "executor.hpp"
#include "tensorio.hpp"

using namespace deepx;

#define DXE_API extern "C" __attribute__((visibility("default")))

static size_t copy_out(const std::string &s, char *buf, size_t buflen) {
    if (buf && buflen) {
        size_t n = s.size() < buflen - 1 ? s.size() : buflen - 1;
        std::memcpy(buf, s.data(), n);
        buf[n] = '\0';
    }
    return s.size();
}

DXE_API void *dxe_create(void) { try { return new Executor(); } catch (...) { return nullptr; } }
DXE_API void dxe_destroy(void *ex) { delete static_cast<Executor *>(ex); }
// executes one IR line; writes the reply line; returns the reply length (may exceed buflen)
DXE_API size_t dxe_execute(void *ex, const char *line, char *reply, size_t buflen) {
    return copy_out(static_cast<Executor *>(ex)->execute(line ? line : ""), reply, buflen);
}
// executes the newline-separated IR lines of `text` as one batch (what the UDP server does with a
// datagram); writes the replies joined by '\n'; returns their total length
DXE_API size_t dxe_execute_batch(void *ex, const char *text, char *reply, size_t buflen) {
    std::vector<std::string> lines;
    std::istringstream in(text ? text : "");
    std::string line;
    while (std::getline(in, line)) if (!line.empty()) lines.push_back(line);
    if (lines.empty()) return copy_out("", reply, buflen);
    std::string out;
    for (const std::string &r : static_cast<Executor *>(ex)->execute_batch(lines)) { if (!out.empty()) out += '\n'; out += r; }
    return copy_out(out, reply, buflen);
}
// wait for the device before every reply (the DEEPX_SYNC switch; default off = reply at launch, like op-cuda)
DXE_API void dxe_set_sync(void *ex, int on) { static_cast<Executor *>(ex)->sync_each = on != 0; }
// graph recording on/off (the DEEPX_GRAPH switch) and the batch counters: "batches captures replays rejects"
DXE_API void dxe_set_graphs(void *ex, int on) { static_cast<Executor *>(ex)->use_graphs = on != 0; }
// one launch for runs of float elementwise lines inside a batch (the DEEPX_FUSE switch), and its counters: "runs lines"
DXE_API void dxe_set_fusion(void *ex, int on) { static_cast<Executor *>(ex)->use_fusion = on != 0; }
// lines that can share a launch are answered at once and held until the run is complete (the DEEPX_DEFER switch);
// dxe_flush launches what is held, dxe_held counts it, dxe_defer_stats: "held_lines flushes"
DXE_API void dxe_set_defer(void *ex, int on) { auto *e = static_cast<Executor *>(ex); if (!on) e->flush(); e->defer = on != 0; }
DXE_API void dxe_flush(void *ex) { static_cast<Executor *>(ex)->flush(); }
DXE_API size_t dxe_held(void *ex) { return static_cast<Executor *>(ex)->held(); }
DXE_API size_t dxe_defer_stats(void *ex, char *out, size_t buflen) {
    const auto &s = static_cast<Executor *>(ex)->stats;
    return copy_out(std::to_string(s.held_lines) + " " + std::to_string(s.flushes), out, buflen);
}
// independent kernel-only lines of a batch on n side streams in turn (the DEEPX_STREAMS switch; 1 = in order on the default stream);
// dxe_side_launches: how many launches went to a side stream so far
DXE_API void dxe_set_streams(void *ex, int n) { static_cast<Executor *>(ex)->streams = n < 1 ? 1 : n > 8 ? 8 : n; }
DXE_API size_t dxe_side_launches(void *ex) { return (size_t)static_cast<Executor *>(ex)->stats.side_launches; }
// tensors allocated from now on take their storage from the library's pool of freed blocks (1, the default; the DEEPX_POOL
// switch) or from the driver each time (0); tensors that exist keep what they have and return it where it came from
// 1 (default): `newtensor` owes its zero fill to the first launch that names the tensor; 0: it fills at once (DEEPX_ZERO_AT_ALLOC=1)
DXE_API void dxe_set_zero_later(void *ex, int on) { static_cast<Executor *>(ex)->mem.zero_later = on != 0; }
DXE_API void dxe_set_pool(int on) { deepx::tensor_pool_enabled() = on != 0; }
DXE_API size_t dxe_fusion_stats(void *ex, char *out, size_t buflen) {
    const auto &s = static_cast<Executor *>(ex)->stats;
    return copy_out(std::to_string(s.fused_runs) + " " + std::to_string(s.fused_lines) + " " + std::to_string(s.matmul_groups) + " " + std::to_string(s.matmul_lines), out, buflen);
}
// host-time breakdown of execute() (see Executor::Profile): on/off, and "lines parse match run sync reply" in ns; reading resets
DXE_API void dxe_set_profile(void *ex, int on) { static_cast<Executor *>(ex)->profile = on != 0; }
DXE_API size_t dxe_profile(void *ex, char *out, size_t buflen) {
    auto &p = static_cast<Executor *>(ex)->prof;
    const std::string s = std::to_string(p.lines) + " " + std::to_string(p.parse_ns) + " " + std::to_string(p.match_ns) + " " +
                          std::to_string(p.run_ns) + " " + std::to_string(p.sync_ns) + " " + std::to_string(p.reply_ns);
    p = Executor::Profile{};
    return copy_out(s, out, buflen);
}
DXE_API size_t dxe_stats(void *ex, char *out, size_t buflen) {
    const auto &s = static_cast<Executor *>(ex)->stats;
    return copy_out(std::to_string(s.batches) + " " + std::to_string(s.graph_captures) + " " + std::to_string(s.graph_replays) + " " +
                    std::to_string(s.graph_rejects), out, buflen);
}
// parse + print round trip (no execution): "name(args)->(returns) //metadata", or "error: ..."
DXE_API size_t dxe_parse(const char *line, char *out, size_t buflen) {
    try {
        TF tf(line ? line : "");
        return copy_out(tf.to_string(true), out, buflen);
    } catch (const std::exception &e) {
        return copy_out(std::string("error: ") + e.what(), out, buflen);
    }
}
// which registered signature a call resolves to: "author|signature", or "none: <reason>"
DXE_API size_t dxe_match(void *ex, const char *line, char *out, size_t buflen) {
    try {
        TF call(line ? line : "");
        std::string why;
        auto tf = static_cast<Executor *>(ex)->factory.get_tf(call, &why);
        if (!tf) return copy_out("none: " + why, out, buflen);
        // report the REGISTERED signature: look it up again without cloning the call's metadata
        const auto &fam = static_cast<Executor *>(ex)->factory.families.at(call.name);
        auto ait = fam.by_author.find(call.metadata.author);
        const std::string author = ait == fam.by_author.end() ? fam.author_order.front() : call.metadata.author;
        for (const auto &r : fam.by_author.at(author))
            if (TfFactory::signature_matches(call, *r)) return copy_out(author + "|" + r->to_string(), out, buflen);
        return copy_out("none", out, buflen);
    } catch (const std::exception &e) {
        return copy_out(std::string("error: ") + e.what(), out, buflen);
    }
}
DXE_API size_t dxe_op_table(void *ex, const char *executor_name, char *out, size_t buflen) {
    return copy_out(static_cast<Executor *>(ex)->factory.print_markdown(executor_name ? executor_name : "op-mem-hip"), out, buflen);
}
DXE_API size_t dxe_typedef_roundtrip(const char *text, char *out, size_t buflen) {
    TypeDef t = typedef_from(text ? text : "");
    return copy_out(typedef_str(t) + " " + std::to_string((int)t.category) + " " + std::to_string((int)t.precision), out, buflen);
}
// whether `print` accepts a format for a floating (is_float != 0) or integer tensor: 1 or 0
DXE_API int dxe_print_format_ok(const char *fmt, int is_float) { return print_format_ok(fmt ? fmt : "", is_float != 0) ? 1 : 0; }
// tensor metadata as the reference's .shape YAML; "error: ..." if the tensor does not exist
DXE_API size_t dxe_tensor_yaml(void *ex, const char *name, char *out, size_t buflen) {
    try {
        return copy_out(static_cast<Executor *>(ex)->mem.gettensor(name)->shape.to_yaml(), out, buflen);
    } catch (const std::exception &e) {
        return copy_out(std::string("error: ") + e.what(), out, buflen);
    }
}
DXE_API size_t dxe_shape_yaml_roundtrip(const char *yaml, char *out, size_t buflen) {
    try {
        return copy_out(Shape::from_yaml(yaml).to_yaml(), out, buflen);
    } catch (const std::exception &e) {
        return copy_out(std::string("error: ") + e.what(), out, buflen);
    }
}
// the host side of a tensor's raw `.data` file (tensorio.hpp), without a tensor: "" or "error: ..."
DXE_API size_t dxe_data_write(const char *path, const char *data, size_t bytes, char *out, size_t buflen) {
    try { write_exact(path ? path : "", data, bytes); return copy_out("", out, buflen); }
    catch (const std::exception &e) { return copy_out(std::string("error: ") + e.what(), out, buflen); }
}
DXE_API size_t dxe_data_read(const char *path, char *data, size_t bytes, char *out, size_t buflen) {
    try {
        const HostBytes got = read_exact(path ? path : "", bytes);
        if (bytes) std::memcpy(data, got.data(), bytes);
        return copy_out("", out, buflen);
    } catch (const std::exception &e) { return copy_out(std::string("error: ") + e.what(), out, buflen); }
}
// shape inference helpers by name, result as space-separated ints or "error: ...":
//   transpose(a=shape, b=order) broadcast(a, b) indexselect(a=input, b=index shape, extra=axis)
//   repeat(a=shape, b=repeats) checked_dims(a=shape, b=dims) reduced(a=shape, b=checked dims, extra=keepdims)
//   concat2(a, b, extra=axis) matmul(a, b)
DXE_API size_t dxe_infer_shape(const char *op, const int *a, int na, const int *b, int nb, int extra, char *out, size_t buflen) {
    try {
        std::vector<int> A(a, a + na), B(b, b + nb), r;
        std::string o = op ? op : "";
        if (o == "transpose") r = transpose_shape(A, B);
        else if (o == "broadcast") r = broadcast_shape(A, B);
        else if (o == "indexselect") r = indexselect_shape(A, B, extra);
        else if (o == "repeat") r = repeat_shape(A, B);
        else if (o == "checked_dims") r = checked_dims(A, B);
        else if (o == "reduced") r = reduced_shape(A, B, extra != 0);
        else if (o == "concat2") r = concat_shape({A, B}, extra);
        else if (o == "matmul") r = matmul_shape(A, B);
        else return copy_out("error: unknown op", out, buflen);
        std::string s;
        for (size_t i = 0; i < r.size(); ++i) s += (i ? " " : "") + std::to_string(r[i]);
        return copy_out(s, out, buflen);
    } catch (const std::exception &e) {
        return copy_out(std::string("error: ") + e.what(), out, buflen);
    }
}
