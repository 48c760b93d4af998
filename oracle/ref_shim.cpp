// ref_shim.cpp — C entry points around the REFERENCE's own deepxcore sources, compiled where they
// lie under the reference checkout by ref.mk into oracle/_ref/libdeepxref.so.
//
// TEST INFRASTRUCTURE ONLY (used by tests/ to pin the executor's protocol layer against the real
// reference): IR parsing and printing (tf/tf.cpp), dtype strings (dtype.hpp), op matching
// (tf/tffactory.cpp) and the shape-inference helpers that do not need Shape's constructor
// (shape_changeshape.cpp, shape_reduce.cpp), and the raw file I/O behind tensor `.data` files
// (stdutil/fs.cpp).  This file contains no reference code; it only calls it.
// The arithmetic headers of op-ompsimd are NOT buildable here (Highway, OpenBLAS, jemalloc and
// yaml-cpp are absent), nor is deepxcore/shape.cpp (yaml-cpp); functions that need them are
// dropped by the linker's section garbage collection and never called.
#include <cstring>
#include <sstream>
#include <string>
#include <vector>
#include "deepx/dtype.hpp"
#include "deepx/shape_changeshape.hpp"
#include "deepx/shape_reduce.hpp"
#include "deepx/tf/tf.hpp"
#include "deepx/tf/tffactory.hpp"
#include "stdutil/fs.hpp"

#define REF_API extern "C" __attribute__((visibility("default")))

static size_t put(const std::string &s, char *out, size_t n) {
    if (out && n) { size_t k = s.size() < n - 1 ? s.size() : n - 1; std::memcpy(out, s.data(), k); out[k] = 0; }
    return s.size();
}
static std::string ints(const std::vector<int> &v) {
    std::ostringstream o;
    for (size_t i = 0; i < v.size(); ++i) o << (i ? " " : "") << v[i];
    return o.str();
}

REF_API size_t ref_parse(const char *line, char *out, size_t n) {
    try {
        deepx::tf::TF tf;
        tf.metadata.id = 0;
        tf.metadata.created_at = tf.metadata.sent_at = tf.metadata.recv_at = std::chrono::system_clock::time_point::min();
        tf.parse(line);
        return put(tf.to_string(true), out, n);
    } catch (const std::exception &e) { return put(std::string("error: ") + e.what(), out, n); }
}
REF_API size_t ref_typedef(const char *text, char *out, size_t n) {
    deepx::TypeDef t = deepx::dtype(text);
    return put(deepx::dtype_str(t) + " " + std::to_string((int)t.category()) + " " + std::to_string((int)t.precision()), out, n);
}
// registered: newline-separated "author|signature line" rows registered in order; returns the
// to_string() of the TF get_tf picks for `call`, or "none"
REF_API size_t ref_match(const char *registered, const char *call, char *out, size_t n) {
    try {
        deepx::tf::TfFactory f;
        std::istringstream in(registered);
        std::string row;
        while (std::getline(in, row)) {
            if (row.empty()) continue;
            size_t bar = row.find('|');
            auto tf = std::make_shared<deepx::tf::TF>();
            tf->metadata.id = 0;
            tf->parse(row.substr(bar + 1));
            tf->metadata.author = row.substr(0, bar);
            // the reference registers precision unions as Precision bit-ors in C++ (tfs.cpp); its
            // text parser has no union syntax, so rebuild the masks from the printed signature
            auto fix = [](deepx::tf::Param &p, const std::string &sig_param) {
                size_t lt = sig_param.find('<'), gt = sig_param.find('>');
                if (lt == std::string::npos || gt == std::string::npos) return;
                std::string prec = sig_param.substr(lt + 1, gt - lt - 1);
                if (prec.find('|') == std::string::npos) return;
                uint16_t bits = 0;
                std::istringstream ws(prec);
                std::string w;
                while (std::getline(ws, w, '|')) bits |= (uint16_t)deepx::precision(w);
                p.dtype.parts.precision = (deepx::Precision)bits;
            };
            std::string sig = row.substr(bar + 1);
            size_t arrow = sig.find(")->(");
            std::string a = sig.substr(sig.find('(') + 1, arrow - sig.find('(') - 1), r = sig.substr(arrow + 4);
            auto split = [](const std::string &s) {
                std::vector<std::string> out;
                std::istringstream is(s);
                std::string item;
                while (std::getline(is, item, ',')) if (item.find_first_not_of(" )") != std::string::npos) out.push_back(item);
                return out;
            };
            auto as = split(a), rs = split(r);
            for (size_t i = 0; i < as.size() && i < tf->args.size(); ++i) fix(tf->args[i], as[i]);
            for (size_t i = 0; i < rs.size() && i < tf->returns.size(); ++i) fix(tf->returns[i], rs[i]);
            f.add_tf(tf);
        }
        deepx::tf::TF c;
        c.metadata.id = 0;
        c.parse(call);
        auto got = f.get_tf(c);
        return put(got ? got->to_string(false, true) : std::string("none"), out, n);
    } catch (const std::exception &e) { return put(std::string("error: ") + e.what(), out, n); }
}
REF_API size_t ref_transpose_shape(const int *shape, int ndim, const int *order, char *out, size_t n) {
    try { return put(ints(deepx::transposeShape(std::vector<int>(shape, shape + ndim), std::vector<int>(order, order + ndim))), out, n); }
    catch (const std::exception &e) { return put(std::string("error: ") + e.what(), out, n); }
}
REF_API size_t ref_broadcast_shape(const int *a, int na, const int *b, int nb, char *out, size_t n) {
    return put(ints(deepx::broadcastShape(std::vector<int>(a, a + na), std::vector<int>(b, b + nb))), out, n);
}
REF_API size_t ref_indexselect_shape(const int *in, int nin, const int *idx, int nidx, int axis, char *out, size_t n) {
    return put(ints(deepx::indexselectShape(std::vector<int>(in, in + nin), std::vector<int>(idx, idx + nidx), axis)), out, n);
}
REF_API size_t ref_repeat_shape(const int *in, int nin, const int *reps, int nreps, char *out, size_t n) {
    try { return put(ints(deepx::repeatShape(std::vector<int>(in, in + nin), std::vector<int>(reps, reps + nreps))), out, n); }
    catch (const std::exception &e) { return put(std::string("error: ") + e.what(), out, n); }
}
REF_API size_t ref_checked_dims(const int *shape, int ndim, const int *dims, int ndims, char *out, size_t n) {
    try { return put(ints(deepx::checkedDims(std::vector<int>(shape, shape + ndim), std::vector<int>(dims, dims + ndims))), out, n); }
    catch (const std::exception &e) { return put(std::string("error: ") + e.what(), out, n); }
}
REF_API size_t ref_reduced_shape(const int *shape, int ndim, const int *dims, int ndims, int keepdims, char *out, size_t n) {
    return put(ints(deepx::reducedShape(std::vector<int>(shape, shape + ndim), std::vector<int>(dims, dims + ndims), keepdims != 0)), out, n);
}

// stdutil/fs.cpp: the writer and the two readers of a tensor's raw `.data` file.  Each returns ""
// or the text of the exception.
REF_API size_t ref_fs_save(const char *path, const unsigned char *data, size_t bytes, char *out, size_t n) {
    try { stdutil::save(data, bytes, path); return put("", out, n); }
    catch (const std::exception &e) { return put(std::string("error: ") + e.what(), out, n); }
}
REF_API size_t ref_fs_load(const char *path, unsigned char *data, size_t bytes, char *out, size_t n) {
    try { stdutil::load(path, data, bytes); return put("", out, n); }
    catch (const std::exception &e) { return put(std::string("error: ") + e.what(), out, n); }
}
// the size-agnostic reader: the file's size, then min(size, bytes) bytes into data
REF_API size_t ref_fs_load_any(const char *path, unsigned char *data, size_t bytes, char *out, size_t n) {
    try {
        auto got = stdutil::load(path);
        std::memcpy(data, got.second.get(), got.first < bytes ? got.first : bytes);
        return put(std::to_string(got.first), out, n);
    } catch (const std::exception &e) { return put(std::string("error: ") + e.what(), out, n); }
}
REF_API size_t ref_fs_filename(const char *path, char *out, size_t n) { return put(stdutil::filename(path), out, n); }
