// ops.cpp — the executor's op table: every deepxIR op, its registered signature and the host
// wrapper that turns a parsed instruction into one C-ABI kernel call.
//
// The table is the union of the reference executors' registrations
// (executor/op-ompsimd/src/client/tfs.cpp:19-689, executor/op-cuda/src/client/tfs.cpp:20-646; the
// generated lists docs/executor/op-mem-{ompsimd,cuda}/list.md): same op names, authors, tftypes,
// argument order, categories and precision masks, so front/py dispatches unchanged.  Where the
// reference has one TF class per op (executor/op-ompsimd/src/deepx/tf/*.hpp), this file has one
// table row per op and a handful of wrapper templates keyed by the C-ABI function they call.
//
// Behaviour kept from the reference wrappers: dtype is read from the STORED tensors, mismatches
// give "Type mismatch: a != b"; a missing tensor gives "tensor not found: <name>"; scalars are
// T(std::stof(text)) or a named arg (tf.hpp:84-125); vectors are "[3 4 5]" (tf.hpp:127-158).
// The wrapper defects listed against op-ompsimd (PowScalar/MinScalar reading the dtype from the
// scalar, RSubScalar reading the scalar from the tensor slot) are NOT reproduced: the registered
// signature and the front's emission order (front/py/deepx/nn/functional/rtf_*.py) are the contract.
#include <algorithm>
#include <cctype>
#include <cmath>
#include <cstdio>
#include <cstring>
#include <fstream>
#include <functional>
#include <iostream>
#include "factory.hpp"
#include "mem.hpp"
#include "tensorio.hpp"

namespace deepx {

namespace {

using RunFn = std::function<int(const TF &, Mem &, std::string &)>;

class OpTF : public TF {
public:
    std::string formula;
    RunFn fn;
    int run(Mem &mem, std::string &error) override {
        try {
            return fn(*this, mem, error);
        } catch (const std::exception &e) {  // the reference lets these kill the process; here they become error replies
            error = e.what();
            return 1;
        }
    }
    std::string math_formula() const override { return formula; }
    std::shared_ptr<TF> clone() const override { return std::make_shared<OpTF>(*this); }
};

void reg(TfFactory &f, const char *name, const char *author, const char *tftype, const char *formula,
         std::initializer_list<const char *> args, std::initializer_list<const char *> returns, RunFn fn) {
    auto tf = std::make_shared<OpTF>();
    tf->name = name;
    tf->metadata.author = author;
    tf->tftype = tftype;
    tf->formula = formula;
    auto registered = [](const char *text) {  // "type:name" with precision unions allowed
        std::string t = text;
        size_t colon = t.find(':');
        Param p;
        p.dtype = typedef_union_from(t.substr(0, colon));
        p.textvalue = t.substr(colon + 1);
        return p;
    };
    for (const char *a : args) tf->args.push_back(registered(a));
    for (const char *r : returns) tf->returns.push_back(registered(r));
    tf->fn = std::move(fn);
    const std::string kind = tftype, op = name;
    static const struct { const char *name; int code, kind; } chainable[] = {
        {"add", DXH_CHAIN_ADD, 1}, {"sub", DXH_CHAIN_SUB, 1}, {"mul", DXH_CHAIN_MUL, 1}, {"div", DXH_CHAIN_DIV, 1},
        {"max", DXH_CHAIN_MAX, 1}, {"min", DXH_CHAIN_MIN, 1},
        {"addscalar", DXH_CHAIN_ADDSCALAR, 2}, {"subscalar", DXH_CHAIN_SUBSCALAR, 2}, {"rsubscalar", DXH_CHAIN_RSUBSCALAR, 3},
        {"mulscalar", DXH_CHAIN_MULSCALAR, 2}, {"divscalar", DXH_CHAIN_DIVSCALAR, 2}, {"rdivscalar", DXH_CHAIN_RDIVSCALAR, 3},
        {"maxscalar", DXH_CHAIN_MAXSCALAR, 2}, {"minscalar", DXH_CHAIN_MINSCALAR, 2},
        {"sqrt", DXH_CHAIN_SQRT, 4}, {"exp", DXH_CHAIN_EXP, 4}, {"log", DXH_CHAIN_LOG, 4}};
    if (kind == "elementwise")
        for (const auto &c : chainable)
            if (op == c.name) { tf->chain_code = c.code; tf->chain_kind = c.kind; }
    // lines that only dxh_chain_rows takes: the cast, the square, a vector spread over rows or columns
    if (op == "todtype") { tf->chain_code = DXH_CHAIN_COPY; tf->chain_kind = 5; }
    if (op == "broadcastTo") { tf->chain_code = DXH_CHAIN_COPY; tf->chain_kind = 6; }
    if (op == "powscalar") { tf->chain_code = DXH_CHAIN_SQUARE; tf->chain_kind = 7; }
    if (op == "sum") { tf->chain_code = DXH_CHAIN_ROWSUM; tf->chain_kind = 8; }
    if (op == "reducemax") { tf->chain_code = DXH_CHAIN_ROWMAX; tf->chain_kind = 8; }
    if (op == "reducemin") { tf->chain_code = DXH_CHAIN_ROWMIN; tf->chain_kind = 8; }
    tf->graph_safe = kind == "elementwise" || kind == "reduce" || kind == "changeshape" || op == "matmul" ||
                     op == "constant" || op == "arange";
    if (op == "reshape") tf->graph_safe = false;  // rewrites the tensor's shape on the host
    tf->overwrites_results = tf->graph_safe || op == "uniform" || op == "normal" || op == "copytensor" || op == "loadtensordata";
    f.add_tf(tf);
}

// ---- argument access -------------------------------------------------------------------------
std::shared_ptr<Tensor> tensor_of(const Param &p, Mem &mem) { return mem.gettensor(p.textvalue); }

int fail(std::string &error, const std::string &msg) { error = msg; return 1; }
int hip_result(int rc, const char *op, std::string &error) {
    if (rc == DXH_OK) return 0;
    if (rc == DXH_ERR_DTYPE) return fail(error, std::string("Unsupported dtype for ") + op);
    return fail(error, std::string(op) + ": " + dxh_error_string(rc));
}

// T(std::stof(text)) for every T when the text parses as a float, else a named arg (tf.hpp:119-124)
dxh_scalar scalar_of(const Param &p, Mem &mem) {
    dxh_scalar s{0.0, 0};
    if (text_is_float(p.textvalue)) {
        float v = std::stof(p.textvalue);
        s.f = (double)v;
        if (std::isnan(v)) s.i = 0;
        else if (v >= 9.2233720368547758e18f) s.i = INT64_MAX;
        else if (v <= -9.2233720368547758e18f) s.i = INT64_MIN;
        else s.i = (int64_t)v;
        return s;
    }
    if (!mem.existarg(p.textvalue)) throw std::runtime_error("arg not found: " + p.textvalue);
    const ArgValue &a = mem.getarg(p.textvalue);
    if (auto v = std::get_if<int32_t>(&a)) { s.f = *v; s.i = *v; }
    else if (auto v = std::get_if<int64_t>(&a)) { s.f = (double)*v; s.i = *v; }
    else if (auto v = std::get_if<float>(&a)) { s.f = *v; s.i = (int64_t)*v; }
    else if (auto v = std::get_if<double>(&a)) { s.f = *v; s.i = (int64_t)*v; }
    else if (auto v = std::get_if<bool>(&a)) { s.f = *v; s.i = *v; }
    else throw std::runtime_error("arg is not a number: " + p.textvalue);
    return s;
}
int int_of(const Param &p, Mem &mem) { return (int)scalar_of(p, mem).i; }
float float_of(const Param &p, Mem &mem) { return (float)scalar_of(p, mem).f; }

bool bool_of(const Param &p) {
    std::string v = p.textvalue;
    std::transform(v.begin(), v.end(), v.begin(), [](unsigned char c) { return std::tolower(c); });
    if (v == "true") return true;
    if (v == "false") return false;
    throw std::invalid_argument("Invalid bool value:" + p.textvalue);
}
std::vector<std::string> words_of(const Param &p) {
    std::string t = p.textvalue;
    size_t a = t.find_first_not_of("[]"), b = t.find_last_not_of("[]");
    t = a == std::string::npos ? "" : t.substr(a, b - a + 1);
    std::vector<std::string> out;
    std::istringstream in(t);
    std::string w;
    while (in >> w) out.push_back(w);
    return out;
}
// "[3 4 5]" -> ints; an empty list is an error like tf.hpp:146-150; a bare name looks up a vecset vector
std::vector<int> ints_of(const Param &p, Mem &mem) {
    auto words = words_of(p);
    if (words.empty()) throw std::invalid_argument("Invalid argument index");
    if (words.size() == 1 && !text_is_float(words[0]) && mem.existarg(words[0])) {
        const ArgValue &a = mem.getarg(words[0]);
        std::vector<int> out;
        if (auto v = std::get_if<std::vector<int32_t>>(&a)) out.assign(v->begin(), v->end());
        else if (auto v = std::get_if<std::vector<int64_t>>(&a)) out.assign(v->begin(), v->end());
        else throw std::runtime_error("arg is not an int vector: " + words[0]);
        return out;
    }
    std::vector<int> out;
    for (auto &w : words) out.push_back((int)std::stof(w));
    return out;
}

bool same_dtype(std::initializer_list<const Tensor *> ts, std::string &error) {
    const Tensor *first = *ts.begin();
    bool ok = true;
    for (const Tensor *t : ts) ok &= t->shape.dtype == first->shape.dtype;
    if (!ok) {
        error = "Type mismatch: ";
        bool lead = true;
        for (const Tensor *t : ts) { if (!lead) error += " != "; error += precision_str(t->shape.dtype); lead = false; }
    }
    return ok;
}
bool same_size(std::initializer_list<const Tensor *> ts, std::string &error) {
    const Tensor *first = *ts.begin();
    for (const Tensor *t : ts)
        if (t->shape.size != first->shape.size) { error = "shape mismatch: " + dims_str(first->shape.shape) + " vs " + dims_str(t->shape.shape); return false; }
    return true;
}

// ---- wrapper templates -----------------------------------------------------------------------
using BinaryFn = int (*)(int, const void *, const void *, void *, int64_t, void *);
using ScalarFn = int (*)(int, const void *, dxh_scalar, void *, int64_t, void *);
using RScalarFn = int (*)(int, dxh_scalar, const void *, void *, int64_t, void *);
using UnaryFn = int (*)(int, const void *, void *, int64_t, void *);

RunFn binary(BinaryFn f, const char *op) {  // (A, B) -> (C)
    return [f, op](const TF &c, Mem &mem, std::string &error) {
        auto A = tensor_of(c.args[0], mem), B = tensor_of(c.args[1], mem), C = tensor_of(c.returns[0], mem);
        if (!same_dtype({A.get(), B.get(), C.get()}, error) || !same_size({A.get(), B.get(), C.get()}, error)) return 1;
        return hip_result(f(A->dtype(), A->data, B->data, C->data, C->shape.size, mem.stream), op, error);
    };
}
RunFn with_scalar(ScalarFn f, const char *op) {  // (A, scalar) -> (C)
    return [f, op](const TF &c, Mem &mem, std::string &error) {
        auto A = tensor_of(c.args[0], mem), C = tensor_of(c.returns[0], mem);
        if (!same_dtype({A.get(), C.get()}, error) || !same_size({A.get(), C.get()}, error)) return 1;
        return hip_result(f(A->dtype(), A->data, scalar_of(c.args[1], mem), C->data, C->shape.size, mem.stream), op, error);
    };
}
RunFn with_rscalar(RScalarFn f, const char *op) {  // (scalar, A) -> (C)
    return [f, op](const TF &c, Mem &mem, std::string &error) {
        auto A = tensor_of(c.args[1], mem), C = tensor_of(c.returns[0], mem);
        if (!same_dtype({A.get(), C.get()}, error) || !same_size({A.get(), C.get()}, error)) return 1;
        return hip_result(f(A->dtype(), scalar_of(c.args[0], mem), A->data, C->data, C->shape.size, mem.stream), op, error);
    };
}
RunFn unary(UnaryFn f, const char *op) {  // (A) -> (C)
    return [f, op](const TF &c, Mem &mem, std::string &error) {
        auto A = tensor_of(c.args[0], mem), C = tensor_of(c.returns[0], mem);
        if (!same_dtype({A.get(), C.get()}, error) || !same_size({A.get(), C.get()}, error)) return 1;
        return hip_result(f(A->dtype(), A->data, C->data, C->shape.size, mem.stream), op, error);
    };
}
bool mask_ok(const Tensor &m, std::string &error) {
    if (m.shape.dtype != Precision::Bool) { error = "mask must be a bool tensor, got " + precision_str(m.shape.dtype); return false; }
    return true;
}
using CmpEpsFn = int (*)(int, const void *, const void *, float, void *, int64_t, void *);
using CmpEpsScalarFn = int (*)(int, const void *, dxh_scalar, float, void *, int64_t, void *);
RunFn compare_eps(CmpEpsFn f, const char *op) {  // (A, B, epsilon) -> (mask)
    return [f, op](const TF &c, Mem &mem, std::string &error) {
        auto A = tensor_of(c.args[0], mem), B = tensor_of(c.args[1], mem), M = tensor_of(c.returns[0], mem);
        if (!same_dtype({A.get(), B.get()}, error) || !mask_ok(*M, error) || !same_size({A.get(), B.get(), M.get()}, error)) return 1;
        return hip_result(f(A->dtype(), A->data, B->data, float_of(c.args[2], mem), M->data, M->shape.size, mem.stream), op, error);
    };
}
RunFn compare_eps_scalar(CmpEpsScalarFn f, const char *op) {  // (A, scalar, epsilon) -> (mask)
    return [f, op](const TF &c, Mem &mem, std::string &error) {
        auto A = tensor_of(c.args[0], mem), M = tensor_of(c.returns[0], mem);
        if (!mask_ok(*M, error) || !same_size({A.get(), M.get()}, error)) return 1;
        return hip_result(f(A->dtype(), A->data, scalar_of(c.args[1], mem), float_of(c.args[2], mem), M->data, M->shape.size, mem.stream), op, error);
    };
}
RunFn compare(BinaryFn f, const char *op) {  // (A, B) -> (mask)
    return [f, op](const TF &c, Mem &mem, std::string &error) {
        auto A = tensor_of(c.args[0], mem), B = tensor_of(c.args[1], mem), M = tensor_of(c.returns[0], mem);
        if (!same_dtype({A.get(), B.get()}, error) || !mask_ok(*M, error) || !same_size({A.get(), B.get(), M.get()}, error)) return 1;
        return hip_result(f(A->dtype(), A->data, B->data, M->data, M->shape.size, mem.stream), op, error);
    };
}
RunFn compare_scalar(ScalarFn f, const char *op) {  // (A, scalar) -> (mask)
    return [f, op](const TF &c, Mem &mem, std::string &error) {
        auto A = tensor_of(c.args[0], mem), M = tensor_of(c.returns[0], mem);
        if (!mask_ok(*M, error) || !same_size({A.get(), M.get()}, error)) return 1;
        return hip_result(f(A->dtype(), A->data, scalar_of(c.args[1], mem), M->data, M->shape.size, mem.stream), op, error);
    };
}

using ReduceFn = int (*)(int, const void *, const int32_t *, int, const int32_t *, int, void *, void *, size_t, void *);
RunFn reduce(ReduceFn f, const char *op) {  // (A, vector dims, bool keepdims) -> (B)
    return [f, op](const TF &c, Mem &mem, std::string &error) {
        auto A = tensor_of(c.args[0], mem), B = tensor_of(c.returns[0], mem);
        std::vector<int> dims = checked_dims(A->shape.shape, ints_of(c.args[1], mem));
        const bool keepdims = bool_of(c.args[2]);
        if (!same_dtype({A.get(), B.get()}, error)) return 1;
        std::vector<int> want = reduced_shape(A->shape.shape, dims, keepdims);
        if (Shape(want).size != B->shape.size)
            return fail(error, "Shape mismatch: reduced shape " + dims_str(want) + " vs output " + dims_str(B->shape.shape));
        size_t need = 0;
        int rc = dxh_reduce_workspace_bytes(A->dtype(), A->shape.shape.data(), A->shape.dim(), dims.data(), (int)dims.size(), &need);
        if (rc != DXH_OK) return hip_result(rc, op, error);
        void *ws = need ? mem.workspace(need) : nullptr;
        return hip_result(f(A->dtype(), A->data, A->shape.shape.data(), A->shape.dim(), dims.data(), (int)dims.size(), B->data, ws,
                            need ? mem.workspace_bytes() : 0, mem.stream), op, error);
    };
}

// "T1 = zeros(shape)", as op-cuda's newtensor documents itself (its storage is whatever cudaMalloc returns).  The fill is
// made here, on the NULL stream, or owed (`zero_later`): then whoever launches the first kernel that names the tensor makes
// it, or drops it when that kernel overwrites the whole tensor anyway (Executor::settle).
std::shared_ptr<Tensor> new_tensor(const std::vector<int> &shape, Precision p, bool zero_later) {
    for (int d : shape) if (d < 0) throw std::invalid_argument("negative dimension in shape " + dims_str(shape));
    if (shape.empty()) throw std::invalid_argument("newtensor: empty shape");
    auto t = std::make_shared<Tensor>(shape, p);
    if (zero_later) t->zero_pending = true;
    else dxh_check(t->fill_zero(nullptr), "newtensor zero fill");
    return t;
}

}  // namespace

int register_all(TfFactory &f) {
    // ---- tensorlife (tf/tensorlife.hpp) ---------------------------------------------------------
    auto newtensor = [](const TF &c, Mem &mem, std::string &error) {
        const TypeDef &t = c.returns[0].dtype;
        if ((uint8_t(t.category) & uint8_t(DataCategory::Tensor)) == 0) return fail(error, "newtensor: return type must include tensor category");
        if (precision_bytes(t.precision) == 0) return fail(error, "newtensor: unsupported precision " + precision_str(t.precision));
        if (t.precision == Precision::Float8E5M2 || t.precision == Precision::Float8E4M3)
            return fail(error, "newtensor: " + precision_str(t.precision) + " has not been implemented");
        auto tensor = new_tensor(ints_of(c.args[0], mem), t.precision, mem.zero_later);
        if (!mem.addtensor(c.returns[0].textvalue, tensor)) std::cerr << "tensor already exists: " << c.returns[0].textvalue << std::endl;
        return 0;
    };
    reg(f, "newtensor", "", "tensorlife", "T1 = zeros(shape)", {"vector<int32>:shape"}, {"tensor<any>:t"}, newtensor);
    reg(f, "newtensor", "", "tensorlife", "T1 = zeros(shape)", {"var<string>:shape"}, {"tensor<any>:t"}, newtensor);
    reg(f, "copytensor", "", "tensorlife", "T2.data = T1.data", {"tensor<any>:src"}, {"tensor<any>:dst"},
        [](const TF &c, Mem &mem, std::string &error) {
            auto S = tensor_of(c.args[0], mem), D = tensor_of(c.returns[0], mem);
            if (S->shape.dtype != D->shape.dtype) return fail(error, "copytensor: input type and return type must be the same");
            if (!same_size({S.get(), D.get()}, error)) return 1;
            return hip_result(dxh_memcpy_d2d(D->data, S->data, (size_t)S->shape.bytes(), mem.stream), "copytensor", error);
        });
    reg(f, "deltensor", "", "tensorlife", "del->T1", {}, {"tensor<any>:t"},
        [](const TF &c, Mem &mem, std::string &) { mem.delete_tensor(c.returns[0].textvalue); return 0; });
    reg(f, "renametensor", "", "tensorlife", "rename(newname)->T1", {"var<string>:new_name"}, {"tensor<any>:t"},
        [](const TF &c, Mem &mem, std::string &) { mem.rename_tensor(c.returns[0].textvalue, c.args[0].textvalue); return 0; });

    // ---- arg (tf/arg.hpp) -----------------------------------------------------------------------
    reg(f, "argset", "", "arg", "argvalue->argname", {"var<any>:value"}, {"var<any>:name"},
        [](const TF &c, Mem &mem, std::string &error) {
            const TypeDef &t = c.returns[0].dtype;
            if ((uint8_t(t.category) & uint8_t(DataCategory::Var)) == 0) return fail(error, "datatype must be var");
            const std::string &v = c.args[0].textvalue, &name = c.returns[0].textvalue;
            switch (t.precision) {
            case Precision::Int32: mem.setarg(name, (int32_t)std::atoi(v.c_str())); break;
            case Precision::Int64: mem.setarg(name, (int64_t)std::stoll(v)); break;
            case Precision::Float32: mem.setarg(name, std::stof(v)); break;
            case Precision::Float64: mem.setarg(name, std::stod(v)); break;
            case Precision::Bool: mem.setarg(name, bool_of(c.args[0])); break;
            case Precision::String: mem.setarg(name, v); break;
            default: return fail(error, "Unsupported dtype: " + typedef_str(c.args[0].dtype));
            }
            return 0;
        });
    reg(f, "vecset", "", "arg", "[3  4  5]->shape", {"vector<any>:value"}, {"vector<any>:name"},
        [](const TF &c, Mem &mem, std::string &error) {
            const TypeDef &t = c.returns[0].dtype;
            if ((uint8_t(t.category) & uint8_t(DataCategory::Vector)) == 0) return fail(error, "datatype must be vector");
            auto words = words_of(c.args[0]);
            const std::string &name = c.returns[0].textvalue;
            switch (t.precision) {
            case Precision::Int64: { std::vector<int64_t> v; for (auto &w : words) v.push_back(std::stoll(w)); mem.setarg(name, v); break; }
            case Precision::Int32: case Precision::Int16: case Precision::Int8: {
                std::vector<int32_t> v; for (auto &w : words) v.push_back(std::stoi(w)); mem.setarg(name, v); break; }
            case Precision::Float64: { std::vector<double> v; for (auto &w : words) v.push_back(std::stod(w)); mem.setarg(name, v); break; }
            case Precision::Float32: { std::vector<float> v; for (auto &w : words) v.push_back(std::stof(w)); mem.setarg(name, v); break; }
            case Precision::String: mem.setarg(name, words); break;
            default: return fail(error, "Unsupported dtype: " + typedef_str(t));
            }
            return 0;
        });

    // ---- init (tf/init.hpp) ----------------------------------------------------------------------
    reg(f, "constant", "miaobyte", "init", "constant(value)->T1", {"var<any>:value"}, {"tensor<any>:t"},
        [](const TF &c, Mem &mem, std::string &error) {
            auto T = tensor_of(c.returns[0], mem);
            dxh_scalar v = T->shape.dtype == Precision::Bool && !text_is_float(c.args[0].textvalue)
                               ? dxh_scalar{bool_of(c.args[0]) ? 1.0 : 0.0, bool_of(c.args[0]) ? 1 : 0} : scalar_of(c.args[0], mem);
            return hip_result(dxh_constant(T->dtype(), T->data, T->shape.size, v, mem.stream), "constant", error);
        });
    reg(f, "arange", "miaobyte", "init", "arange(start,step)->T1", {"var<any>:start", "var<any>:step"}, {"tensor<any>:t"},
        [](const TF &c, Mem &mem, std::string &error) {
            auto T = tensor_of(c.returns[0], mem);
            return hip_result(dxh_arange(T->dtype(), T->data, T->shape.size, scalar_of(c.args[0], mem), scalar_of(c.args[1], mem), mem.stream), "arange", error);
        });
    reg(f, "uniform", "miaobyte", "init", "uniform(low,high,seed)->T1", {"var<any>:low", "var<any>:high", "var<int32>:seed"}, {"tensor<any>:t"},
        [](const TF &c, Mem &mem, std::string &error) {
            auto T = tensor_of(c.returns[0], mem);
            return hip_result(dxh_uniform(T->dtype(), T->data, T->shape.size, scalar_of(c.args[0], mem), scalar_of(c.args[1], mem),
                                          (uint32_t)int_of(c.args[2], mem), mem.stream), "uniform", error);
        });
    reg(f, "normal", "miaobyte", "init", "normal(mean,stddev,seed)->T1", {"var<any>:mean", "var<any>:stddev", "var<int32>:seed"}, {"tensor<any>:t"},
        [](const TF &c, Mem &mem, std::string &error) {
            auto T = tensor_of(c.returns[0], mem);
            return hip_result(dxh_normal(T->dtype(), T->data, T->shape.size, scalar_of(c.args[0], mem), scalar_of(c.args[1], mem),
                                         (uint32_t)int_of(c.args[2], mem), mem.stream), "normal", error);
        });
    reg(f, "dropout", "miaobyte", "init", "dropout(p,seed)->A", {"var<float32>:p", "var<int32>:seed"}, {"tensor<any>:A"},
        [](const TF &c, Mem &mem, std::string &error) {
            auto T = tensor_of(c.returns[0], mem);
            return hip_result(dxh_dropout(T->dtype(), T->data, T->shape.size, float_of(c.args[0], mem), (uint32_t)int_of(c.args[1], mem), mem.stream), "dropout", error);
        });

    // ---- io (tf/io.hpp) --------------------------------------------------------------------------
    auto print = [](const TF &c, Mem &mem, std::string &error) {
        if (!mem.existstensor(c.args[0].textvalue)) return fail(error, "print " + c.args[0].textvalue + " not found");
        auto T = tensor_of(c.args[0], mem);
        print_tensor(*T, c.args.size() > 1 ? c.args[1].textvalue : std::string(), std::cout);
        return 0;
    };
    reg(f, "print", "miaobyte", "io", "print(T1)", {"tensor<any>:t"}, {}, print);
    reg(f, "print", "miaobyte", "io", "print(T1)", {"tensor<any>:t", "var<string>:format"}, {}, print);
    reg(f, "save", "", "io", "save(T1,path)", {"tensor<any>:t", "var<string>:path"}, {},
        [](const TF &c, Mem &mem, std::string &error) {
            if (!mem.existstensor(c.args[0].textvalue)) return fail(error, "save " + c.args[0].textvalue + " not found");
            save_tensor(*tensor_of(c.args[0], mem), c.args[1].textvalue);
            return 0;
        });
    reg(f, "load", "", "io", "load(path)", {"var<string>:path"}, {},
        [](const TF &c, Mem &mem, std::string &) {
            auto [name, tensor] = load_tensor(c.args[0].textvalue);
            if (mem.existstensor(name)) mem.delete_tensor(name);  // the reference replaces with a warning
            mem.addtensor(name, tensor);
            return 0;
        });
    reg(f, "loadtensordata", "", "io", "loadtensordata(path)->tensor", {"var<string>:path"}, {"tensor<any>:t"},
        [](const TF &c, Mem &mem, std::string &error) {
            if (!mem.existstensor(c.returns[0].textvalue)) return fail(error, "loadtensordata " + c.returns[0].textvalue + " not found");
            load_tensor_data(c.args[0].textvalue, *tensor_of(c.returns[0], mem));
            return 0;
        });

    // ---- elementwise (tf/elementwise.hpp; op-cuda tf/elementwise_*.hpp) ---------------------------
    reg(f, "todtype", "", "elementwise", "T3(dtypeA)->T1(dtypeB)", {"tensor<any>:A"}, {"tensor<any>:C"},
        [](const TF &c, Mem &mem, std::string &error) {
            auto A = tensor_of(c.args[0], mem), C = tensor_of(c.returns[0], mem);
            if (A->shape.size != C->shape.size) return fail(error, "Shape mismatch: " + std::to_string(A->shape.size) + " != " + std::to_string(C->shape.size));
            return hip_result(dxh_todtype(A->dtype(), A->data, C->dtype(), C->data, C->shape.size, mem.stream), "todtype", error);
        });
#define T_ANY "tensor<any>"
    reg(f, "add", "miaobyte", "elementwise", "T3=T1+T2", {T_ANY ":a", T_ANY ":b"}, {T_ANY ":c"}, binary(dxh_add, "add"));
    // the reference registers a second author for add (cblas / cublas); both names reach the same kernel
    reg(f, "add", "cublas", "elementwise", "T3=T1+T2", {T_ANY ":a", T_ANY ":b"}, {T_ANY ":c"}, binary(dxh_add, "add"));
    reg(f, "add", "cblas", "elementwise", "T3=T1+T2", {T_ANY ":a", T_ANY ":b"}, {T_ANY ":c"}, binary(dxh_add, "add"));
    reg(f, "addscalar", "miaobyte", "elementwise", "T3=T1+scalar", {T_ANY ":a", "var<any>:scalar"}, {T_ANY ":c"}, with_scalar(dxh_addscalar, "addscalar"));
    reg(f, "sub", "miaobyte", "elementwise", "T3=T1-T2", {T_ANY ":a", T_ANY ":b"}, {T_ANY ":c"}, binary(dxh_sub, "sub"));
    reg(f, "subscalar", "miaobyte", "elementwise", "T3=T1-scalar", {T_ANY ":a", "var<any>:scalar"}, {T_ANY ":c"}, with_scalar(dxh_subscalar, "subscalar"));
    reg(f, "rsubscalar", "miaobyte", "elementwise", "T3=scalar-T1", {"var<any>:scalar", T_ANY ":a"}, {T_ANY ":c"}, with_rscalar(dxh_rsubscalar, "rsubscalar"));
    reg(f, "mul", "miaobyte", "elementwise", "T3=T1*T2", {T_ANY ":A", T_ANY ":B"}, {T_ANY ":C"}, binary(dxh_mul, "mul"));
    reg(f, "mulscalar", "miaobyte", "elementwise", "T3=T1*scalar", {T_ANY ":A", "var<any>:b"}, {T_ANY ":C"}, with_scalar(dxh_mulscalar, "mulscalar"));
    reg(f, "div", "miaobyte", "elementwise", "T3=T1/T2", {T_ANY ":A", T_ANY ":B"}, {T_ANY ":C"}, binary(dxh_div, "div"));
    reg(f, "divscalar", "miaobyte", "elementwise", "T3=T1/scalar", {T_ANY ":A", "var<any>:scalar"}, {T_ANY ":C"}, with_scalar(dxh_divscalar, "divscalar"));
    reg(f, "rdivscalar", "miaobyte", "elementwise", "T3=scalar/T1", {"var<any>:scalar", T_ANY ":A"}, {T_ANY ":C"}, with_rscalar(dxh_rdivscalar, "rdivscalar"));
    reg(f, "invert", "miaobyte", "elementwise", "T3=~T1", {"tensor<int64|int32|int16|int8|bool>:A"}, {"tensor<int64|int32|int16|int8|bool>:C"}, unary(dxh_invert, "invert"));
    reg(f, "sqrt", "miaobyte", "elementwise", "T3=sqrt(T1)", {T_ANY ":A"}, {T_ANY ":C"}, unary(dxh_sqrt, "sqrt"));
    reg(f, "pow", "miaobyte", "elementwise", "T3=T1^T2", {T_ANY ":A", T_ANY ":B"}, {T_ANY ":C"}, binary(dxh_pow, "pow"));
    reg(f, "powscalar", "miaobyte", "elementwise", "T3=T1^scalar", {T_ANY ":A", "var<any>:scalar"}, {T_ANY ":C"}, with_scalar(dxh_powscalar, "powscalar"));
    reg(f, "rpowscalar", "miaobyte", "elementwise", "T3=scalar^T1", {"var<any>:scalar", T_ANY ":A"}, {T_ANY ":C"}, with_rscalar(dxh_rpowscalar, "rpowscalar"));
    reg(f, "log", "miaobyte", "elementwise", "T3=log(T1)", {T_ANY ":A"}, {T_ANY ":C"}, unary(dxh_log, "log"));
    reg(f, "exp", "miaobyte", "elementwise", "T3=exp(T1)", {T_ANY ":A"}, {T_ANY ":C"}, unary(dxh_exp, "exp"));
    reg(f, "sin", "miaobyte", "elementwise", "T3=sin(T1)", {T_ANY ":A"}, {T_ANY ":C"}, unary(dxh_sin, "sin"));
    reg(f, "cos", "miaobyte", "elementwise", "T3=cos(T1)", {T_ANY ":A"}, {T_ANY ":C"}, unary(dxh_cos, "cos"));
    reg(f, "tan", "miaobyte", "elementwise", "T3=tan(T1)", {T_ANY ":A"}, {T_ANY ":C"}, unary(dxh_tan, "tan"));
    reg(f, "max", "miaobyte", "elementwise", "T3=max(T1,T2)", {T_ANY ":A", T_ANY ":B"}, {T_ANY ":C"}, binary(dxh_max, "max"));
    reg(f, "maxscalar", "miaobyte", "elementwise", "T3=max(T1,scalar)", {T_ANY ":A", "var<any>:scalar"}, {T_ANY ":C"}, with_scalar(dxh_maxscalar, "maxscalar"));
    reg(f, "min", "miaobyte", "elementwise", "T3=min(T1,T2)", {T_ANY ":A", T_ANY ":B"}, {T_ANY ":C"}, binary(dxh_min, "min"));
    reg(f, "minscalar", "miaobyte", "elementwise", "T3=min(T1,scalar)", {T_ANY ":A", "var<any>:scalar"}, {T_ANY ":C"}, with_scalar(dxh_minscalar, "minscalar"));
    reg(f, "equal", "miaobyte", "elementwise", "equal(T1,T2)->mask", {T_ANY ":A", T_ANY ":B", "var<float32>:epsilon"}, {"tensor<bool>:mask"}, compare_eps(dxh_equal, "equal"));
    reg(f, "equalscalar", "miaobyte", "elementwise", "mask=equal(T1,scalar)", {T_ANY ":A", "var<any>:scalar", "var<float32>:epsilon"}, {"tensor<bool>:mask"}, compare_eps_scalar(dxh_equalscalar, "equalscalar"));
    reg(f, "notequal", "miaobyte", "elementwise", "notequal(T1,T2)->mask", {T_ANY ":A", T_ANY ":B", "var<float32>:epsilon"}, {"tensor<bool>:mask"}, compare_eps(dxh_notequal, "notequal"));
    reg(f, "notequalscalar", "miaobyte", "elementwise", "mask=notequal(T1,scalar)", {T_ANY ":A", "var<any>:scalar", "var<float32>:epsilon"}, {"tensor<bool>:mask"}, compare_eps_scalar(dxh_notequalscalar, "notequalscalar"));
    reg(f, "less", "miaobyte", "elementwise", "mask=less(T1,T2)", {T_ANY ":A", T_ANY ":B"}, {"tensor<bool>:mask"}, compare(dxh_less, "less"));
    reg(f, "lessscalar", "miaobyte", "elementwise", "mask=less(T1,scalar)", {T_ANY ":A", "var<any>:scalar"}, {"tensor<bool>:mask"}, compare_scalar(dxh_lessscalar, "lessscalar"));
    reg(f, "greater", "miaobyte", "elementwise", "mask=greater(T1,T2)", {T_ANY ":A", T_ANY ":B"}, {"tensor<bool>:mask"}, compare(dxh_greater, "greater"));
    reg(f, "greaterscalar", "miaobyte", "elementwise", "mask=greater(T1,scalar)", {T_ANY ":A", "var<any>:scalar"}, {"tensor<bool>:mask"}, compare_scalar(dxh_greaterscalar, "greaterscalar"));
    reg(f, "switch", "miaobyte", "elementwise", "C=switch([tensors],case)", {"listtensor<any>:tensors", "tensor<int32|bool>:cases"}, {T_ANY ":C"},
        [](const TF &c, Mem &mem, std::string &error) {
            auto names = words_of(c.args[0]);
            if (names.empty() || names.size() > DXH_SWITCH_MAX) return fail(error, "switch takes 1.." + std::to_string(DXH_SWITCH_MAX) + " tensors");
            auto cases = tensor_of(c.args[1], mem), C = tensor_of(c.returns[0], mem);
            std::vector<std::shared_ptr<Tensor>> ts;
            std::vector<const void *> ptrs;
            for (auto &n : names) {
                ts.push_back(mem.gettensor(n));
                if (ts.back()->shape.dtype != C->shape.dtype) return fail(error, "Type mismatch: " + precision_str(ts.back()->shape.dtype) + " != " + precision_str(C->shape.dtype));
                if (!same_size({ts.back().get(), C.get()}, error)) return 1;
                ptrs.push_back(ts.back()->data);
            }
            if (!same_size({cases.get(), C.get()}, error)) return 1;
            if (cases->shape.dtype == Precision::Bool && names.size() != 2) return fail(error, "For bool cases, tensors size must be 2");
            return hip_result(dxh_switch(C->dtype(), ptrs.data(), (int)ptrs.size(), cases->dtype(), cases->data, C->data, C->shape.size, mem.stream), "switch", error);
        });

    // ---- reduce (tf/reduce.hpp) ------------------------------------------------------------------
    reg(f, "sum", "miaobyte", "reduce", "B = sum(A, axis=[1 2], keepdims=false)", {T_ANY ":A", "vector<int32>:axis", "var<bool>:keepdims"}, {T_ANY ":B"}, reduce(dxh_sum, "sum"));
    reg(f, "prod", "miaobyte", "reduce", "B = prod(A, axis=[1 2], keepdims=false)", {T_ANY ":A", "vector<int32>:axis", "var<bool>:keepdims"}, {T_ANY ":B"}, reduce(dxh_prod, "prod"));
    reg(f, "reducemax", "miaobyte", "reduce", "B = reducemax(A, axis=[1 2], keepdims=false)", {T_ANY ":A", "vector<int32>:axis", "var<bool>:keepdims"}, {T_ANY ":B"}, reduce(dxh_reducemax, "reducemax"));
    reg(f, "reducemin", "miaobyte", "reduce", "B = reducemin(A, axis=[1 2], keepdims=false)", {T_ANY ":A", "vector<int32>:axis", "var<bool>:keepdims"}, {T_ANY ":B"}, reduce(dxh_reducemin, "reducemin"));

    // ---- changeshape (tf/changeshape.hpp) ---------------------------------------------------------
    reg(f, "reshape", "miaobyte", "changeshape", "T1.reshape(shape)->T2", {T_ANY ":A", "vector<int32>:shape"}, {T_ANY ":B"},
        [](const TF &c, Mem &mem, std::string &error) {
            auto A = tensor_of(c.args[0], mem), B = tensor_of(c.returns[0], mem);
            if (!same_dtype({A.get(), B.get()}, error)) return 1;
            std::vector<int> shape = ints_of(c.args[1], mem);
            Shape ns(shape, B->shape.dtype);
            if (ns.size != A->shape.size || ns.size != B->shape.size) return fail(error, "Shape size mismatch");
            B->shape = ns;  // metadata only when A and B are the same tensor, else a copy too
            if (A->data != B->data) return hip_result(dxh_memcpy_d2d(B->data, A->data, (size_t)A->shape.bytes(), mem.stream), "reshape", error);
            return 0;
        });
    reg(f, "transpose", "miaobyte", "changeshape", "T1.transpose(dimorder=[1,0])->T2", {T_ANY ":A", "vector<int32>:dim_order"}, {T_ANY ":C"},
        [](const TF &c, Mem &mem, std::string &error) {
            auto A = tensor_of(c.args[0], mem), C = tensor_of(c.returns[0], mem);
            if (!same_dtype({A.get(), C.get()}, error)) return 1;
            std::vector<int> order = ints_of(c.args[1], mem);
            std::vector<int> want = transpose_shape(A->shape.shape, order);
            if (C->shape.size != A->shape.size) return fail(error, "transpose error!shape");
            if (A->data == C->data) return fail(error, "transpose cannot run in place");
            (void)want;
            return hip_result(dxh_transpose(A->dtype(), A->data, A->shape.shape.data(), A->shape.dim(), order.data(), C->data, mem.stream), "transpose", error);
        });
    reg(f, "concat", "miaobyte", "changeshape", "Tresult = concat([T1, T2...], axis=3)", {"listtensor<any>:tensors", "var<int32>:dim"}, {T_ANY ":result"},
        [](const TF &c, Mem &mem, std::string &error) {
            auto names = words_of(c.args[0]);
            if (names.empty()) return fail(error, "concat needs at least one tensor");
            auto R = tensor_of(c.returns[0], mem);
            int axis = int_of(c.args[1], mem);
            if (axis < 0) axis += R->shape.dim();
            std::vector<std::shared_ptr<Tensor>> ts;
            std::vector<const void *> ptrs;
            std::vector<std::vector<int>> shapes;
            std::vector<int32_t> axis_sizes;
            for (auto &n : names) {
                ts.push_back(mem.gettensor(n));
                if (ts.back()->shape.dtype != R->shape.dtype) return fail(error, "Type mismatch: " + precision_str(ts.back()->shape.dtype) + " != " + precision_str(R->shape.dtype));
                shapes.push_back(ts.back()->shape.shape);
                ptrs.push_back(ts.back()->data);
            }
            std::vector<int> want = concat_shape(shapes, axis);
            if (want != R->shape.shape) return fail(error, "Output tensor shape size must match the sum of input tensor shape sizes for concat");
            for (auto &s : shapes) axis_sizes.push_back(s[axis]);
            return hip_result(dxh_concat(R->dtype(), ptrs.data(), (int)ptrs.size(), axis_sizes.data(), want.data(), (int)want.size(), axis, R->data, mem.stream), "concat", error);
        });
    reg(f, "broadcastTo", "miaobyte", "changeshape", "T2 = T1.broadcastTo(new_shape=[4,3,2])", {T_ANY ":A", "vector<int32>:new_shape"}, {T_ANY ":B"},
        [](const TF &c, Mem &mem, std::string &error) {
            auto A = tensor_of(c.args[0], mem), B = tensor_of(c.returns[0], mem);
            if (!same_dtype({A.get(), B.get()}, error)) return 1;
            std::vector<int> ns = ints_of(c.args[1], mem);
            if (broadcast_shape(A->shape.shape, ns) != ns) return fail(error, "Broadcast shape mismatch");
            if (Shape(ns).size != B->shape.size) return fail(error, "Broadcast shape mismatch: output is " + dims_str(B->shape.shape));
            return hip_result(dxh_broadcastTo(A->dtype(), A->data, A->shape.shape.data(), A->shape.dim(), ns.data(), (int)ns.size(), B->data, mem.stream), "broadcastTo", error);
        });
    reg(f, "indexselect", "miaobyte", "changeshape", "T2 = T1.indexselect(index=T3, axis=3)", {T_ANY ":A", "tensor<int64|int32>:index", "var<int32>:axis"}, {T_ANY ":B"},
        [](const TF &c, Mem &mem, std::string &error) {
            auto A = tensor_of(c.args[0], mem), I = tensor_of(c.args[1], mem), B = tensor_of(c.returns[0], mem);
            if (!same_dtype({A.get(), B.get()}, error)) return 1;
            if (I->shape.dtype != Precision::Int64 && I->shape.dtype != Precision::Int32) return fail(error, "index only support int32 or int64");
            int axis = int_of(c.args[2], mem);
            int ga = axis < 0 ? axis + A->shape.dim() : axis;
            if (ga < 0 || ga >= A->shape.dim()) return fail(error, "Axis is out of bounds");
            if (indexselect_shape(A->shape.shape, I->shape.shape, ga) != B->shape.shape) return fail(error, "Indexselect shape mismatch");
            return hip_result(dxh_indexselect(A->dtype(), A->data, A->shape.shape.data(), A->shape.dim(), I->dtype(), I->data, I->shape.shape.data(),
                                              I->shape.dim(), ga, B->data, mem.stream), "indexselect", error);
        });
    reg(f, "repeat", "miaobyte", "changeshape", "T1.repeat(repeats=[4,3,2])->T2", {T_ANY ":A", "vector<int32>:repeats"}, {T_ANY ":B"},
        [](const TF &c, Mem &mem, std::string &error) {
            auto A = tensor_of(c.args[0], mem), B = tensor_of(c.returns[0], mem);
            if (!same_dtype({A.get(), B.get()}, error)) return 1;
            std::vector<int> reps = ints_of(c.args[1], mem);
            if (repeat_shape(A->shape.shape, reps) != B->shape.shape) return fail(error, "Repeat shape mismatch");
            return hip_result(dxh_repeat(A->dtype(), A->data, A->shape.shape.data(), A->shape.dim(), reps.data(), B->data, mem.stream), "repeat", error);
        });

    // ---- matmul (tf/matmul.hpp).  The front asks for author "cublas" (authormap.py:60), op-ompsimd
    // registers "cblas" and "miaobyte": all three names reach the same MFMA / tiled kernel.
    auto matmul = [](const TF &c, Mem &mem, std::string &error) {
        auto A = tensor_of(c.args[0], mem), B = tensor_of(c.args[1], mem), C = tensor_of(c.returns[0], mem);
        if (!same_dtype({A.get(), B.get(), C.get()}, error)) return 1;
        std::vector<int> want = matmul_shape(A->shape.shape, B->shape.shape);
        if (want != C->shape.shape) return fail(error, "matmul: output shape " + dims_str(C->shape.shape) + " != " + dims_str(want));
        int64_t batch = 1;
        for (int i = 0; i + 2 < A->shape.dim(); ++i) batch *= A->shape.shape[i];
        const int64_t m = A->shape.at(-2), k = A->shape.at(-1), n = B->shape.at(-1);
        size_t need = 0;
        int rc = dxh_matmul_workspace_bytes(A->dtype(), A->data, B->data, C->data, batch, m, k, n, &need);
        if (rc != DXH_OK) return hip_result(rc, "matmul", error);
        void *ws = need ? mem.workspace(need) : nullptr;
        return hip_result(dxh_matmul(A->dtype(), A->data, B->data, C->data, batch, m, k, n, ws, need ? mem.workspace_bytes() : 0, mem.stream), "matmul", error);
    };
    for (const char *author : {"cublas", "cblas", "miaobyte"})
        reg(f, "matmul", author, "matmul", "T3=T1 @ T2", {T_ANY ":A", T_ANY ":B"}, {T_ANY ":C"}, matmul);
#undef T_ANY
    return 0;
}

// ---- several elementwise lines as one launch --------------------------------------------------
namespace {
// A run goes out in one of two forms: tensors of one float dtype and one size through dxh_chain, or,
// when the lines differ in dtype (todtype), square a tensor (powscalar by 2) or spread a [rows, 1] /
// [1, cols] tensor over [rows, cols] (broadcastTo), through dxh_chain_rows.
struct ChainPlan {
    bool by_rows = false;
    int dtype = 0;
    int64_t n = 0, rows = 0, cols = 0;
    std::vector<const void *> inputs;
    std::vector<dxh_chain_op> ops;
    std::vector<dxh_chain_tensor> row_inputs;
    std::vector<dxh_chain_rows_op> row_ops;
};
enum { kChainTodtype = 5, kChainBroadcast = 6, kChainPowscalar = 7, kChainSum = 8 };
// The lines of a run as they are taken in, one at a time: add() checks a line against the lines before it and the tensor
// store and either takes it (true) or leaves everything as it was (false: the run ends before that line).
struct ChainLines {
    struct Input { std::string name; const void *data; int dtype, extent; };
    struct Op { dxh_chain_rows_op op; std::string out_name; };
    std::vector<Input> inputs;
    std::vector<Op> ops;
    bool needs_rows = false, has_f64 = false;
    int64_t rows = 0, cols = 0;
    static bool is_float(int dtype) { return dtype == DXH_F64 || dtype == DXH_F32 || dtype == DXH_F16 || dtype == DXH_BF16; }
    // extent of a tensor in the run's view, or -1
    int extent_of(const Tensor &t) const {
        if (t.shape.size == rows * cols) return (int)DXH_CHAIN_FULL;
        if (rows > 1 && cols > 1 && t.shape.dim() >= 1) {
            if (t.shape.size == cols && t.shape.at(-1) == cols) return (int)DXH_CHAIN_ROW;
            if (t.shape.size == rows && t.shape.at(-1) == 1) return (int)DXH_CHAIN_COLUMN;
        }
        return -1;
    }
    bool add(const TF *tf, Mem &mem, size_t max_ops) {
        if (ops.size() >= max_ops) return false;
        if (!tf || tf->chain_kind == 0 || tf->metadata.benchmark_repeat > 1 || tf->returns.size() != 1) return false;
        const int kind = tf->chain_kind;
        const size_t nargs = kind == 4 || kind == kChainTodtype ? 1 : kind == kChainSum ? 3 : 2;
        if (tf->args.size() != nargs) return false;
        const Param *tensors[2] = {nullptr, nullptr};
        const Param *scalar = nullptr;
        switch (kind) {
        case 1: tensors[0] = &tf->args[0]; tensors[1] = &tf->args[1]; break;
        case 2: case kChainPowscalar: tensors[0] = &tf->args[0]; scalar = &tf->args[1]; break;
        case 3: scalar = &tf->args[0]; tensors[0] = &tf->args[1]; break;
        default: tensors[0] = &tf->args[0]; break;  // unary, todtype, broadcastTo (whose second argument is the shape)
        }
        auto out = mem.findtensor(tf->returns[0].textvalue);
        if (!out || !is_float(out->dtype()) || out->shape.size == 0) return false;
        if (ops.empty()) {  // the view comes from the first line's output, or from its operand when it reduces rows
            auto shaper = out;
            if (kind == kChainSum) shaper = mem.findtensor(tf->args[0].textvalue);
            if (!shaper || shaper->shape.size == 0) return false;
            cols = shaper->shape.dim() >= 1 ? shaper->shape.at(-1) : 1;
            rows = shaper->shape.size / std::max<int64_t>(cols, 1);
        }
        Op op{};
        op.op.code = tf->chain_code;
        op.op.out = out->data;
        op.op.dtype = out->dtype();
        op.op.extent = extent_of(*out);
        op.out_name = tf->returns[0].textvalue;
        if (kind == kChainSum) {
            // the sum / max / min of every row of a [rows, cols] tensor; whether the row stage of the separate
            // reduction is one the fused kernels can stand in for is asked of the library once the run is known
            if (rows < 2 || out->shape.size != rows) return false;
            auto in = mem.findtensor(tf->args[0].textvalue);
            if (!in || in->shape.dim() < 1 || in->shape.at(-1) != cols || in->shape.size != rows * cols) return false;
            try {
                if (checked_dims(in->shape.shape, ints_of(tf->args[1], mem)) != std::vector<int>{in->shape.dim() - 1}) return false;
                (void)bool_of(tf->args[2]);
            } catch (const std::exception &) { return false; }
            op.op.extent = DXH_CHAIN_COLUMN;
        }
        if (op.op.extent < 0) return false;
        bool line_needs_rows = op.op.extent != DXH_CHAIN_FULL || kind >= kChainTodtype || (!ops.empty() && out->dtype() != ops[0].op.dtype);
        if (scalar) {
            try { op.op.scalar = scalar_of(*scalar, mem); } catch (const std::exception &) { return false; }
        }
        if (kind == kChainPowscalar && (op.op.scalar.f != 2.0 || out->dtype() != DXH_F32)) return false;  // only the square has a chain code
        if (kind == kChainBroadcast) {
            std::vector<int> ns;
            try { ns = ints_of(tf->args[1], mem); } catch (const std::exception &) { return false; }
            if (ns != out->shape.shape || op.op.extent != DXH_CHAIN_FULL) return false;
        }
        std::vector<Input> new_inputs;
        bool ok = true;
        for (int side = 0; side < 2 && ok; ++side) {
            if (!tensors[side]) continue;
            const std::string &name = tensors[side]->textvalue;
            auto t = mem.findtensor(name);
            if (!t || !is_float(t->dtype())) { ok = false; break; }
            // A tensor that the run produced has the extent its producing line gave it; only a tensor read
            // from memory is classified by its shape.  The two differ on a square view, where the [rows]
            // result of a row sum without keepdims is a column to the run and looks like a row by shape;
            // a line on such a vector follows its operand.
            int produced_by = -1;
            for (size_t j = ops.size(); j-- > 0;)
                if (ops[j].out_name == name) { produced_by = (int)j; break; }
            const int extent = produced_by >= 0 ? ops[produced_by].op.extent : extent_of(*t);
            if (extent < 0) { ok = false; break; }
            if (kind != kChainBroadcast && kind != kChainSum && extent != DXH_CHAIN_FULL && rows == cols && out->shape.dim() == 1 && out->shape.size == rows)
                op.op.extent = extent;
            // what the line itself would refuse: another dtype (but for todtype), another size (but for broadcastTo)
            if (kind != kChainTodtype && t->dtype() != out->dtype()) { ok = false; break; }
            if (kind == kChainSum && extent != DXH_CHAIN_FULL) { ok = false; break; }
            if (kind != kChainBroadcast && kind != kChainSum && (extent != op.op.extent || t->shape.size != out->shape.size)) { ok = false; break; }
            if (kind == kChainBroadcast && broadcast_shape(t->shape.shape, out->shape.shape) != out->shape.shape) { ok = false; break; }
            line_needs_rows = line_needs_rows || extent != DXH_CHAIN_FULL || t->dtype() != out->dtype();
            int ref = produced_by >= 0 ? DXH_CHAIN_RESULT + produced_by : -1;
            if (ref < 0) {
                for (size_t j = 0; j < inputs.size() && ref < 0; ++j) if (inputs[j].name == name) ref = (int)j;
                for (size_t j = 0; j < new_inputs.size() && ref < 0; ++j) if (new_inputs[j].name == name) ref = (int)(inputs.size() + j);
                if (ref < 0) {
                    if (inputs.size() + new_inputs.size() >= DXH_CHAIN_MAX_INPUTS) { ok = false; break; }
                    ref = (int)(inputs.size() + new_inputs.size());
                    new_inputs.push_back({name, t->data, t->dtype(), extent});
                }
            }
            (side == 0 ? op.op.lhs : op.op.rhs) = ref;
        }
        if (!ok) return false;
        // this line's output is a vector that the run (this line included) reads from memory
        bool overwrites_vector_input = false;
        for (const Input &in : inputs) overwrites_vector_input |= in.extent != DXH_CHAIN_FULL && in.name == op.out_name;
        for (const Input &in : new_inputs) overwrites_vector_input |= in.extent != DXH_CHAIN_FULL && in.name == op.out_name;
        if (overwrites_vector_input) return false;
        const bool line_f64 = out->dtype() == DXH_F64;
        if ((needs_rows || line_needs_rows) && (has_f64 || line_f64)) return false;  // the row form has no fp64
        needs_rows = needs_rows || line_needs_rows;
        has_f64 = has_f64 || line_f64;
        inputs.insert(inputs.end(), new_inputs.begin(), new_inputs.end());
        ops.push_back(op);
        return true;
    }
};
// Builds the longest run starting at tfs[first].  A tensor operand is the latest result of the run
// with that name, else an input of the run (read before the run writes anything, which is what a
// line-by-line execution sees as long as no earlier line of the run has written it — and those are
// taken as results).  A tensor that several lines of the run write is stored by the last of them
// only: nothing reads memory in between.  The first line's output fixes the [rows, cols] view (cols
// = its last dim); later tensors are that size, or a row / column vector of it.  The run ends before
// a line that is not a chainable float op, does not fit the view, needs a ninth input, would overwrite
// a vector that the run reads from memory (lanes of other rows or columns may not have read it yet),
// or whose operands are missing or mismatched (the ordinary path then reports the error for that line).
// structural: stop after the lines have been checked against each other and the tensor store (do the tensors exist,
// do dtypes and extents agree, does the line fit the view) and return how many form a run, without asking whether
// the library would launch it as one: what a caller needs to know before it holds a line back for a later launch.
size_t plan_chain(const std::vector<std::shared_ptr<TF>> &tfs, size_t first, Mem &mem, ChainPlan &plan, size_t max_ops = DXH_CHAIN_ROWS_MAX_OPS, bool structural = false) {
    ChainLines run;
    for (size_t i = first; i < tfs.size(); ++i)
        if (!run.add(tfs[i].get(), mem, max_ops)) break;
    using Input = ChainLines::Input;
    using Op = ChainLines::Op;
    const std::vector<Input> &inputs = run.inputs;
    std::vector<Op> &ops = run.ops;
    const bool needs_rows = run.needs_rows;
    const int64_t rows = run.rows, cols = run.cols;
    const size_t count = ops.size();
    if (count < 2 || structural) return count;
    if (!needs_rows && count > DXH_CHAIN_MAX_OPS) {  // the one-dtype form takes fewer ops
        plan = ChainPlan{};
        return plan_chain(tfs, first, mem, plan, DXH_CHAIN_MAX_OPS);
    }
    for (size_t j = 0; j < count; ++j)
        for (size_t m = j + 1; m < count; ++m)
            if (ops[m].out_name == ops[j].out_name) ops[j].op.out = nullptr;  // overwritten by line m of the run
    plan.by_rows = needs_rows;
    plan.rows = rows; plan.cols = cols;
    if (needs_rows) {
        // whole groups of four columns, tensors aligned to such a group, or the separate calls take it
        bool aligned = cols % 4 == 0;
        auto group_bytes = [](int dtype, int extent) { return (uintptr_t)(extent == DXH_CHAIN_COLUMN ? 1 : 4) * (dtype == DXH_F32 ? 4 : 2); };
        for (const Input &in : inputs) {
            aligned = aligned && (uintptr_t)in.data % group_bytes(in.dtype, in.extent) == 0;
            plan.row_inputs.push_back({in.data, in.dtype, in.extent});
        }
        for (const Op &o : ops) {
            aligned = aligned && (uintptr_t)o.op.out % group_bytes(o.op.dtype, o.op.extent) == 0;  // NULL passes
            plan.row_ops.push_back(o.op);
        }
        if (!aligned) return 0;
        // would the library launch this run?  (Row reductions are the ones it may refuse: their rows must be
        // short enough for one lane group, and 16-bit ones need one of its compiled kernels.)  If not, the
        // run ends before its last row reduction and is asked about again.
        if (dxh_chain_rows_check(plan.row_inputs.data(), (int)plan.row_inputs.size(), plan.row_ops.data(), (int)plan.row_ops.size(), rows, cols) != DXH_OK) {
            size_t last_red = count;
            for (size_t j = 0; j < count; ++j)
                if (ops[j].op.code >= DXH_CHAIN_ROWSUM) last_red = j;
            if (last_red == count || last_red < 2) return 0;
            plan = ChainPlan{};
            return plan_chain(tfs, first, mem, plan, last_red);
        }
        return count;
    }
    plan.dtype = ops[0].op.dtype;
    plan.n = rows * cols;
    for (const Input &in : inputs) plan.inputs.push_back(in.data);
    for (const Op &o : ops) plan.ops.push_back({o.op.code, o.op.lhs, o.op.rhs, o.op.scalar, o.op.out});
    // whole 16-byte vectors at 16-byte aligned addresses, or the separate calls take it
    const int64_t vec = 16 / precision_bytes((Precision)plan.dtype);
    bool aligned = plan.n % vec == 0;
    for (const void *p : plan.inputs) aligned = aligned && ((uintptr_t)p & 15) == 0;
    for (const dxh_chain_op &o : plan.ops) aligned = aligned && ((uintptr_t)o.out & 15) == 0;  // NULL passes
    return aligned ? count : 0;
}
}  // namespace

// ---- consecutive matmul lines on one left operand as one call -------------------------------------
// The front's gated MLP multiplies the same activations by the gate and the up weights in two lines
// (front/py/deepx/nn/modules/mlp/gatedmlp.py:20-26), its attention by the q / k / v weights in three: a
// run of `matmul` lines whose first operand is the same 2-D bf16 / f16 tensor, whose second operands have
// one shape and whose results are distinct tensors that none of the lines reads goes to
// dxh_matmul_shared_a, which launches them together where its kernels allow.  Anything that a single
// line would refuse ends the run before it, so that line reports its own error.
namespace {
// add() takes one more `matmul` line into the run (true) or leaves the run as it was (false: it ends before that line)
struct MatmulGroup {
    std::shared_ptr<Tensor> a;
    std::vector<std::shared_ptr<Tensor>> bs, cs;
    std::vector<std::string> reads, writes;
    bool add(const TF *tf, Mem &mem) {
        if (!tf || tf->name != "matmul" || tf->metadata.benchmark_repeat > 1 || tf->args.size() != 2 || tf->returns.size() != 1) return false;
        auto A = mem.findtensor(tf->args[0].textvalue), B = mem.findtensor(tf->args[1].textvalue), C = mem.findtensor(tf->returns[0].textvalue);
        if (!A || !B || !C || A->shape.dim() != 2 || B->shape.dim() != 2) return false;
        if (A->dtype() != DXH_BF16 && A->dtype() != DXH_F16) return false;
        if (B->dtype() != A->dtype() || C->dtype() != A->dtype()) return false;
        if (A->shape.at(-1) != B->shape.at(-2) || C->shape.shape != std::vector<int>{A->shape.at(-2), B->shape.at(-1)}) return false;
        if (a && (tf->args[0].textvalue != reads[0] || B->shape.shape != bs[0]->shape.shape)) return false;
        const std::string &out = tf->returns[0].textvalue;
        bool clash = out == tf->args[0].textvalue || out == tf->args[1].textvalue;
        for (const std::string &r : reads) clash = clash || r == out;     // an earlier line of the run reads what this one writes
        for (const std::string &w : writes) clash = clash || w == out || w == tf->args[1].textvalue;  // written twice, or read after it was written
        if (clash) return false;
        if (!a) { a = A; reads.push_back(tf->args[0].textvalue); }
        reads.push_back(tf->args[1].textvalue);
        writes.push_back(out);
        bs.push_back(B);
        cs.push_back(C);
        return true;
    }
};
size_t plan_matmul_group(const std::vector<std::shared_ptr<TF>> &tfs, size_t first, Mem &mem, MatmulGroup &g) {
    for (size_t i = first; i < tfs.size(); ++i)
        if (!g.add(tfs[i].get(), mem)) break;
    return g.cs.size();
}
}  // namespace

// ---- a run taken in line by line ----------------------------------------------------------------------
// What run_prefix_length answers for a whole list, kept up to date one line at a time: a caller that holds lines back
// asks for every new line whether it extends what is held, and would otherwise go over all held lines again each time.
struct HeldRun::State {
    ChainLines chain;
    MatmulGroup products;
    bool chain_alive = true, products_alive = true;
    size_t lines = 0;
};
HeldRun::HeldRun() : s_(new State) {}
HeldRun::~HeldRun() = default;
void HeldRun::reset() { s_.reset(new State); }
size_t HeldRun::size() const { return s_->lines; }
bool HeldRun::extend(const TF *tf, Mem &mem) {
    // either form may take the line; a form that refused one is out for the rest of the run (add() leaves a refused
    // line's form untouched, so "refused" must be remembered here)
    const bool c = s_->chain_alive && s_->chain.add(tf, mem, DXH_CHAIN_ROWS_MAX_OPS);
    const bool p = s_->products_alive && s_->products.add(tf, mem);
    if (!c && !p) return false;  // both forms as they were (a line is an elementwise op or a product, never both)
    s_->chain_alive = c;
    s_->products_alive = p;
    ++s_->lines;
    return true;
}

size_t matmul_group_length(const std::vector<std::shared_ptr<TF>> &tfs, size_t first, Mem &mem) {
    MatmulGroup g;
    return plan_matmul_group(tfs, first, mem, g);
}
int run_matmul_group(const std::vector<std::shared_ptr<TF>> &tfs, size_t first, size_t count, Mem &mem, std::string &error) {
    MatmulGroup g;
    if (plan_matmul_group(tfs, first, mem, g) != count || count < 2) return fail(error, "matmul: the run changed between planning and launch");
    std::vector<const void *> bs;
    std::vector<void *> cs;
    for (size_t j = 0; j < count; ++j) { bs.push_back(g.bs[j]->data); cs.push_back(g.cs[j]->data); }
    const int64_t m = g.a->shape.at(-2), k = g.a->shape.at(-1), n = g.bs[0]->shape.at(-1);
    size_t need = 0;
    int rc = dxh_matmul_shared_a_workspace_bytes(g.a->dtype(), g.a->data, bs.data(), cs.data(), (int)count, m, k, n, &need);
    if (rc != DXH_OK) return hip_result(rc, "matmul", error);
    void *ws = need ? mem.workspace(need) : nullptr;
    return hip_result(dxh_matmul_shared_a(g.a->dtype(), g.a->data, bs.data(), cs.data(), (int)count, m, k, n, ws, need ? mem.workspace_bytes() : 0, mem.stream), "matmul", error);
}

size_t chain_length(const std::vector<std::shared_ptr<TF>> &tfs, size_t first, Mem &mem) {
    ChainPlan plan;
    return plan_chain(tfs, first, mem, plan);
}
size_t run_prefix_length(const std::vector<std::shared_ptr<TF>> &tfs, size_t first, Mem &mem) {
    ChainPlan plan;
    const size_t chain = plan_chain(tfs, first, mem, plan, DXH_CHAIN_ROWS_MAX_OPS, true);
    return std::max(chain, matmul_group_length(tfs, first, mem));
}
int run_chain(const std::vector<std::shared_ptr<TF>> &tfs, size_t first, size_t count, Mem &mem, std::string &error) {
    ChainPlan plan;
    if (plan_chain(tfs, first, mem, plan) != count || count < 2) return fail(error, "chain: the run changed between planning and launch");
    if (plan.by_rows)
        return hip_result(dxh_chain_rows(plan.row_inputs.data(), (int)plan.row_inputs.size(), plan.row_ops.data(), (int)plan.row_ops.size(), plan.rows, plan.cols, mem.stream),
                          "chain", error);
    return hip_result(dxh_chain(plan.dtype, plan.inputs.data(), (int)plan.inputs.size(), plan.ops.data(), (int)plan.ops.size(), plan.n, mem.stream),
                      "chain", error);
}

}  // namespace deepx
