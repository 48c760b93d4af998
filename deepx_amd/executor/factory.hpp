// factory.hpp — op registry: name -> author -> implementations, matched by type signature.
//
// Lookup rules follow executor/deepxcore/src/deepx/tf/tffactory.cpp:14-84: unknown op -> none;
// unknown author -> the family's first author; then the first registered TF of that author whose
// arity equals the call's and whose per-parameter category and precision bit sets contain the
// call's (tffactory.hpp:14-31).  The markdown op table mirrors print_markdown (:85-120).
#pragma once
#include <map>
#include <memory>
#include <sstream>
#include <string>
#include <vector>
#include "ir.hpp"

namespace deepx {

class TfFactory {
public:
    struct Family {
        std::vector<std::string> author_order;  // registration order; [0] is the fallback author
        std::map<std::string, std::vector<std::shared_ptr<TF>>> by_author;
    };
    std::map<std::string, Family> families;

    void add_tf(std::shared_ptr<TF> tf) {
        Family &f = families[tf->name];
        if (!f.by_author.count(tf->metadata.author)) f.author_order.push_back(tf->metadata.author);
        f.by_author[tf->metadata.author].push_back(std::move(tf));
    }

    static bool signature_matches(const TF &call, const TF &registered) {
        if (call.args.size() != registered.args.size() || call.returns.size() != registered.returns.size()) return false;
        for (size_t i = 0; i < call.args.size(); ++i)
            if (!call.args[i].dtype.within(registered.args[i].dtype)) return false;
        for (size_t i = 0; i < call.returns.size(); ++i)
            if (!call.returns[i].dtype.within(registered.returns[i].dtype)) return false;
        return true;
    }

    // a clone of the matching implementation carrying the call's metadata, or nullptr;
    // `why` explains a miss
    std::shared_ptr<TF> get_tf(const TF &call, std::string *why = nullptr) const {
        auto fit = families.find(call.name);
        if (fit == families.end()) { if (why) *why = "<op> " + call.name + " not found"; return nullptr; }
        const Family &f = fit->second;
        auto ait = f.by_author.find(call.metadata.author);
        if (ait == f.by_author.end()) ait = f.by_author.find(f.author_order.front());
        for (const auto &tf : ait->second) {
            if (signature_matches(call, *tf)) {
                auto c = tf->clone();
                c->metadata = call.metadata;
                return c;
            }
        }
        if (why) {
            std::ostringstream o;
            o << "<op> " << call.name << " " << call.to_string() << " not found; supported dtypes:";
            for (const auto &tf : ait->second) {
                std::string s = tf->to_string();
                o << " " << s.substr(s.find('('));
            }
            *why = o.str();
        }
        return nullptr;
    }

    static std::string escape_markdown(const std::string &s) {
        std::string out;
        for (char c : s) {
            switch (c) {
            case '\\': out += "\\\\"; break;
            case '"': out += "\\\""; break;
            case '\'': out += "\\'"; break;
            case '\n': out += "\\n"; break;
            case '\t': out += "\\t"; break;
            default: out += c;
            }
        }
        return out;
    }

    std::string print_markdown(const std::string &executor_name) const {
        std::ostringstream ss;
        ss << "## " << executor_name << " 支持算子列表 \n\n";
        ss << "本页面由 `executor/" << executor_name << " 生成，请勿手动修改 \n\n";
        std::map<std::string, std::vector<std::shared_ptr<TF>>> by_type;
        for (const auto &[name, fam] : families)
            for (const auto &author : fam.author_order)
                for (const auto &tf : fam.by_author.at(author)) by_type[tf->tftype].push_back(tf);
        for (const auto &[tftype, tfs] : by_type) {
            ss << "### " << tftype << "\n\n";
            ss << "| Operation | Author |  Math Formula | IR Instruction |\n";
            ss << "|-----------|--------|--------------|----------------|\n";
            for (const auto &tf : tfs) {
                ss << "| " << tf->name << " | " << (tf->metadata.author.empty() ? " none " : tf->metadata.author) << " | "
                   << tf->math_formula() << " | " << escape_markdown(tf->to_string()) << " |\n";
            }
            ss << "\n";
        }
        return ss.str();
    }
};

int register_all(TfFactory &factory);  // ops.cpp
// ops.cpp: how many of the calls tfs[first], tfs[first + 1], ... (nullptr = a line that failed
// earlier) can run as one dxh_chain launch right now (tensors present, one float dtype and size,
// 16-byte aligned whole vectors); 0 or 1 = none.  run_chain launches exactly that run.
size_t chain_length(const std::vector<std::shared_ptr<TF>> &tfs, size_t first, Mem &mem);
int run_chain(const std::vector<std::shared_ptr<TF>> &tfs, size_t first, size_t count, Mem &mem, std::string &error);
// The same for consecutive `matmul` lines that share their first operand (one dxh_matmul_shared_a call).
size_t matmul_group_length(const std::vector<std::shared_ptr<TF>> &tfs, size_t first, Mem &mem);
// How many lines from tfs[first] on belong to one run of either kind, judged by the lines and the tensor store
// alone (1: a line that could start one).  Every such line is known to name existing tensors of matching dtype
// and extent, so holding it back cannot hide an error it would have reported.
size_t run_prefix_length(const std::vector<std::shared_ptr<TF>> &tfs, size_t first, Mem &mem);
// The same question asked one line at a time: extend() takes the line into the run that the lines before it form (as
// one more elementwise line of a chain, or one more product on a shared left operand) and says so, or leaves the run as
// it was and returns false.  A run that has taken n lines is what run_prefix_length would count on those n lines.
class HeldRun {
public:
    HeldRun();
    ~HeldRun();
    void reset();
    size_t size() const;
    bool extend(const TF *tf, Mem &mem);
private:
    struct State;
    std::unique_ptr<State> s_;
};
int run_matmul_group(const std::vector<std::shared_ptr<TF>> &tfs, size_t first, size_t count, Mem &mem, std::string &error);

}  // namespace deepx
