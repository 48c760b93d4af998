// dtype.hpp — deepxIR type vocabulary: data categories, precisions, their text names and the
// subset test used for op matching.  Bit values and names follow
// executor/deepxcore/src/deepx/dtype.hpp:36-146 (enums), :232-247 (match), :266-384 (names), so
// that IR text, `.shape` files and Precision values passed through the C ABI are interchangeable
// with the reference executors.
#pragma once
#include <cstdint>
#include <string>
#include <vector>

namespace deepx {

enum class DataCategory : uint8_t { Unknown = 0, Var = 1, Vector = 2, Tensor = 4, ListTensor = 8 };
inline DataCategory operator|(DataCategory a, DataCategory b) { return DataCategory(uint8_t(a) | uint8_t(b)); }

enum class Precision : uint16_t {
    Float64 = 1 << 0, Float32 = 1 << 1, Float16 = 1 << 2, BFloat16 = 1 << 3,
    Float8E5M2 = 1 << 4, Float8E4M3 = 1 << 5, Float4E2M1 = 1 << 6,
    Int64 = 1 << 8, Int32 = 1 << 9, Int16 = 1 << 10, Int8 = 1 << 11, Int4 = 1 << 12,
    Bool = 1 << 13, String = 1 << 15,
    Any = 0xFFFF,
    Float = 0x007F, Float8 = 0x0030, Int = 0x1F00
};
inline Precision operator|(Precision a, Precision b) { return Precision(uint16_t(a) | uint16_t(b)); }

struct NamedBit { const char *name; uint16_t bit; };
// order = print order of unions
inline const std::vector<NamedBit> &precision_bits_table() {
    static const std::vector<NamedBit> t = {
        {"float64", 1 << 0}, {"float32", 1 << 1}, {"float16", 1 << 2}, {"bfloat16", 1 << 3},
        {"float8e5m2", 1 << 4}, {"float8e4m3", 1 << 5}, {"float4e2m1", 1 << 6},
        {"int64", 1 << 8}, {"int32", 1 << 9}, {"int16", 1 << 10}, {"int8", 1 << 11}, {"int4", 1 << 12},
        {"bool", 1 << 13}, {"string", 1 << 15}};
    return t;
}
inline const std::vector<NamedBit> &category_bits_table() {
    static const std::vector<NamedBit> t = {{"tensor", 4}, {"vector", 2}, {"var", 1}, {"listtensor", 8}};
    return t;
}

// bytes per element of a storable precision, 0 otherwise
inline int precision_bytes(Precision p) {
    switch (p) {
    case Precision::Float64: case Precision::Int64: return 8;
    case Precision::Float32: case Precision::Int32: return 4;
    case Precision::Float16: case Precision::BFloat16: case Precision::Int16: return 2;
    case Precision::Float8E5M2: case Precision::Float8E4M3: case Precision::Int8: case Precision::Bool: return 1;
    default: return 0;
    }
}

inline std::string join_bits(const std::vector<NamedBit> &table, uint16_t value, const char *none) {
    std::string out;
    for (const auto &nb : table)
        if (value & nb.bit) { if (!out.empty()) out += "|"; out += nb.name; }
    return out.empty() ? none : out;
}
inline std::string precision_str(Precision p) {
    if (p == Precision::Any) return "any";
    return join_bits(precision_bits_table(), uint16_t(p), "any");
}
inline std::string category_str(DataCategory c) { return join_bits(category_bits_table(), uint8_t(c), "unknown"); }

inline std::vector<std::string> split_bar(const std::string &s) {
    std::vector<std::string> parts;
    size_t start = 0;
    while (true) {
        size_t bar = s.find('|', start);
        parts.push_back(s.substr(start, bar == std::string::npos ? std::string::npos : bar - start));
        if (bar == std::string::npos) break;
        start = bar + 1;
    }
    return parts;
}

// one precision word; unknown words mean "any" (dtype.hpp:321-364)
inline Precision precision_word(const std::string &w) {
    for (const auto &nb : precision_bits_table()) if (w == nb.name) return Precision(nb.bit);
    if (w == "int") return Precision::Int;
    if (w == "float") return Precision::Float;
    if (w == "float8") return Precision::Float8;
    return Precision::Any;
}
// On the wire the reference's precision() takes a single word, so a union such as
// "float64|float32" is an unknown word and means "any" (dtype.hpp:321-364) — kept as is.
inline Precision precision_from(const std::string &s) { return precision_word(s); }
// Registration side only: the op table is written with unions ("int64|int32|bool"), which the
// reference builds from Precision bit-ors in C++ (tfs.cpp) and prints in this form.
inline Precision precision_union_from(const std::string &s) {
    if (s.find('|') == std::string::npos) return precision_word(s);
    uint16_t bits = 0;
    for (const auto &w : split_bar(s)) bits |= uint16_t(precision_word(w));
    return Precision(bits);
}
inline DataCategory category_from(const std::string &s) {
    uint8_t bits = 0;
    for (const auto &w : split_bar(s))
        for (const auto &nb : category_bits_table()) if (w == nb.name) bits |= uint8_t(nb.bit);
    return DataCategory(bits);
}

struct TypeDef {
    DataCategory category = DataCategory::Unknown;
    Precision precision = Precision::Any;
    TypeDef() = default;
    TypeDef(DataCategory c, Precision p) : category(c), precision(p) {}
    bool operator==(const TypeDef &o) const { return category == o.category && precision == o.precision; }
    // true when every category bit and every precision bit of *this is also set in `registered`
    // (dtype.hpp:232-247: the call's bits must be a subset of the registered signature's)
    bool within(const TypeDef &registered) const {
        uint8_t c = uint8_t(category), rc = uint8_t(registered.category);
        uint16_t p = uint16_t(precision), rp = uint16_t(registered.precision);
        return (c & rc) == c && (p & rp) == p;
    }
};

// "tensor<float32>" -> TypeDef; no <...> means precision any (dtype.hpp:367-384)
inline TypeDef typedef_from(const std::string &s) {
    size_t lt = s.find('<'), gt = s.find('>');
    if (lt == std::string::npos || gt == std::string::npos) return TypeDef(category_from(s), Precision::Any);
    return TypeDef(category_from(s.substr(0, lt)), precision_from(s.substr(lt + 1, gt - lt - 1)));
}
inline TypeDef typedef_union_from(const std::string &s) {
    size_t lt = s.find('<'), gt = s.find('>');
    if (lt == std::string::npos || gt == std::string::npos) return TypeDef(category_from(s), Precision::Any);
    return TypeDef(category_from(s.substr(0, lt)), precision_union_from(s.substr(lt + 1, gt - lt - 1)));
}
inline std::string typedef_str(const TypeDef &t) { return category_str(t.category) + "<" + precision_str(t.precision) + ">"; }

}  // namespace deepx
