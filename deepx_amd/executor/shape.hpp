// shape.hpp — tensor metadata and shape inference of the executor.
//
// Shape{dtype, shape, strides, size} with row-major contiguous strides is the reference's
// in-memory tensor metadata (executor/deepxcore/src/deepx/shape.hpp:44-85, shape.cpp:21-32); on
// disk it is the `<path>.shape` YAML with keys dtype/dim/shape/stride/size (shape.cpp:93-120).
// Shape inference follows executor/deepxcore/src/deepx/shape_changeshape.cpp, shape_reduce.cpp and
// shape_matmul.cpp.
#pragma once
#include <algorithm>
#include <cstdint>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>
#include "dtype.hpp"

namespace deepx {

struct Shape {
    Precision dtype = Precision::Any;
    std::vector<int> shape;
    std::vector<int> strides;
    int64_t size = 0;

    Shape() = default;
    explicit Shape(const std::vector<int> &dims, Precision p = Precision::Any) : dtype(p) { set(dims); }
    void set(const std::vector<int> &dims) {
        shape = dims;
        strides.assign(dims.size(), 1);
        int64_t s = 1;
        for (int i = (int)dims.size() - 1; i >= 0; --i) { strides[i] = (int)s; s *= dims[i]; }
        size = dims.empty() ? 0 : s;
    }
    int dim() const { return (int)shape.size(); }
    int at(int i) const { return shape[i < 0 ? i + dim() : i]; }
    int64_t bytes() const { return size * precision_bytes(dtype); }

    // the five flat keys, emitted in block style like yaml-cpp does for the reference
    std::string to_yaml() const {
        std::ostringstream o;
        o << "dtype: " << precision_str(dtype) << "\n";
        o << "dim: " << dim() << "\n";
        auto seq = [&](const char *key, const std::vector<int> &v) {
            o << key << ":";
            if (v.empty()) { o << " []\n"; return; }
            o << "\n";
            for (int x : v) o << "  - " << x << "\n";
        };
        seq("shape", shape);
        seq("stride", strides);
        o << "size: " << size << "\n";
        return o.str();
    }

    // Accepts block sequences ("- 3") and flow sequences ("[3, 4]"), in any key order, which
    // covers yaml-cpp's output and PyYAML's (front/py/deepx/tensor/shape.py:185-191).
    // Validates shape/stride/size against each other like shape.cpp:102-120.
    static Shape from_yaml(const std::string &text) {
        Shape s;
        std::vector<int> shape, stride;
        int64_t size = -1;
        bool have_dtype = false, have_shape = false, have_stride = false;
        std::istringstream in(text);
        std::string line, key;
        auto trim = [](std::string v) {
            size_t a = v.find_first_not_of(" \t\r"), b = v.find_last_not_of(" \t\r");
            return a == std::string::npos ? std::string() : v.substr(a, b - a + 1);
        };
        auto parse_flow = [&](std::string v, std::vector<int> &out) {
            for (char &c : v) if (c == '[' || c == ']' || c == ',') c = ' ';
            std::istringstream is(v);
            long x;
            while (is >> x) out.push_back((int)x);
        };
        while (std::getline(in, line)) {
            std::string t = trim(line);
            if (t.empty() || t[0] == '#' || t == "---") continue;
            if (t[0] == '-') {  // block sequence item of the current key
                std::string v = trim(t.substr(1));
                if (key == "shape") shape.push_back(std::stoi(v));
                else if (key == "stride") stride.push_back(std::stoi(v));
                continue;
            }
            size_t colon = t.find(':');
            if (colon == std::string::npos) throw std::runtime_error("shape yaml: bad line: " + t);
            key = trim(t.substr(0, colon));
            std::string v = trim(t.substr(colon + 1));
            if (key == "dtype") { s.dtype = precision_from(v); have_dtype = true; }
            else if (key == "shape") { have_shape = true; if (!v.empty()) parse_flow(v, shape); }
            else if (key == "stride") { have_stride = true; if (!v.empty()) parse_flow(v, stride); }
            else if (key == "size") size = std::stoll(v);
        }
        if (!have_dtype || !have_shape) throw std::runtime_error("shape yaml: missing dtype or shape");
        Shape checked(shape, s.dtype);
        if (have_stride && checked.strides != stride) throw std::runtime_error("Shape::fromYaml: strides mismatch");
        if (size >= 0 && checked.size != size) throw std::runtime_error("Shape::fromYaml: size mismatch");
        return checked;
    }
};

inline std::string dims_str(const std::vector<int> &v) {
    std::string s = "[";
    for (size_t i = 0; i < v.size(); ++i) { if (i) s += " "; s += std::to_string(v[i]); }
    return s + "]";
}

// ---- changeshape (shape_changeshape.cpp) -------------------------------------------------------
inline std::vector<int> transpose_shape(const std::vector<int> &shape, const std::vector<int> &order) {
    if (order.size() != shape.size()) throw std::invalid_argument("dimOrder size does not match the number of dimensions");
    std::vector<int> out(shape.size());
    std::vector<bool> seen(shape.size(), false);
    for (size_t i = 0; i < order.size(); ++i) {
        int d = order[i];
        if (d < 0 || d >= (int)shape.size() || seen[d]) throw std::invalid_argument("dimOrder is not a permutation");
        seen[d] = true;
        out[i] = shape[d];
    }
    return out;
}
inline std::vector<int> concat_shape(const std::vector<std::vector<int>> &shapes, int axis) {
    if (shapes.empty()) throw std::invalid_argument("concat needs at least one tensor");
    std::vector<int> out = shapes[0];
    if (axis < 0 || axis >= (int)out.size()) throw std::invalid_argument("concat axis out of range");
    for (size_t t = 1; t < shapes.size(); ++t) {
        if (shapes[t].size() != out.size()) throw std::invalid_argument("All tensors must have the same number of dimensions.");
        for (size_t j = 0; j < out.size(); ++j) {
            if ((int)j == axis) out[j] += shapes[t][j];
            else if (shapes[t][j] != out[j]) throw std::invalid_argument("Shapes of tensors must match except in the concatenation axis.");
        }
    }
    return out;
}
// numpy trailing-aligned broadcast; empty result = not broadcastable (shape_changeshape.cpp:59-78)
inline std::vector<int> broadcast_shape(const std::vector<int> &a, const std::vector<int> &b) {
    size_t n = std::max(a.size(), b.size());
    std::vector<int> out(n);
    for (size_t i = 1; i <= n; ++i) {
        int x = i <= a.size() ? a[a.size() - i] : 1;
        int y = i <= b.size() ? b[b.size() - i] : 1;
        if (x != y && x != 1 && y != 1) return {};
        out[n - i] = std::max(x, y);
    }
    return out;
}
// TF-gather: the index dims replace `axis` (shape_changeshape.cpp:124-144)
inline std::vector<int> indexselect_shape(const std::vector<int> &in, const std::vector<int> &index, int axis) {
    std::vector<int> out(in.begin(), in.begin() + axis);
    out.insert(out.end(), index.begin(), index.end());
    out.insert(out.end(), in.begin() + axis + 1, in.end());
    return out;
}
inline std::vector<int> repeat_shape(const std::vector<int> &in, const std::vector<int> &reps) {
    if (in.size() != reps.size()) throw std::invalid_argument("Shape and repeats must have the same number of dimensions");
    std::vector<int> out(in.size());
    for (size_t i = 0; i < in.size(); ++i) out[i] = in[i] * reps[i];
    return out;
}

// ---- reduce (shape_reduce.cpp) -----------------------------------------------------------------
inline std::vector<int> checked_dims(const std::vector<int> &shape, const std::vector<int> &dims) {
    std::vector<int> out;
    if (dims.empty()) {
        for (int i = 0; i < (int)shape.size(); ++i) out.push_back(i);
        return out;
    }
    for (int d : dims) {
        if (d < 0) d += (int)shape.size();
        if (d < 0 || d >= (int)shape.size()) throw std::invalid_argument("Dimension out of range in sum");
        out.push_back(d);
    }
    std::sort(out.begin(), out.end());
    out.erase(std::unique(out.begin(), out.end()), out.end());
    return out;
}
inline std::vector<int> reduced_shape(const std::vector<int> &shape, const std::vector<int> &checked, bool keepdims) {
    std::vector<bool> red(shape.size(), false);
    for (int d : checked) red[d] = true;
    std::vector<int> out;
    for (size_t i = 0; i < shape.size(); ++i) {
        if (!red[i]) out.push_back(shape[i]);
        else if (keepdims) out.push_back(1);
    }
    if (out.empty()) out.push_back(1);
    return out;
}

// ---- matmul (shape_matmul.cpp:7-22, tensorfunc/matmul.hpp:9-27) ------------------------------------
inline std::vector<int> matmul_shape(const std::vector<int> &a, const std::vector<int> &b) {
    if (a.size() < 2 || b.size() < 2) throw std::invalid_argument("A and B must >= 2D tensors");
    if (a.size() != b.size()) throw std::invalid_argument("A and B must have the same rank");
    for (size_t i = 0; i + 2 < a.size(); ++i)
        if (a[i] != b[i]) throw std::invalid_argument("A and B batch dims must match");
    if (a[a.size() - 1] != b[b.size() - 2]) throw std::invalid_argument("A[-1] must be equal to B[-2]");
    std::vector<int> out = a;
    out.back() = b.back();
    return out;
}

}  // namespace deepx
