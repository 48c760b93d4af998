// tensorio.hpp — tensor files and printing.
//
// A saved tensor is two files (executor/deepxcore/src/deepx/shape.cpp:93-143,
// executor/deepxcore/src/stdutil/fs.cpp:18-50, executor/op-cuda/src/deepx/tensorfunc/io_miaobyte.hpp):
//   <path>.shape  YAML {dtype, dim, shape, stride, size}
//   <path>.data   raw little-endian contiguous elements (bf16/f16 as their 16-bit patterns,
//                 front/py/deepxutil/torch/io.py:11-12)
// The tensor's name on load is the file stem (shape.cpp:140-142).  Device data moves through
// one staged host copy.  print follows executor/deepxcore/src/stdutil/print.hpp:80-129.
#pragma once
#include <cctype>
#include <cstdio>
#include <cstring>
#include <fcntl.h>
#include <sys/mman.h>
#include <sys/stat.h>
#include <unistd.h>
#include <fstream>
#include <memory>
#include <ostream>
#include <string>
#include <vector>
#include "mem.hpp"

namespace deepx {

inline std::string file_stem(const std::string &path) {
    std::string name = path.substr(path.find_last_of('/') + 1);
    size_t dot = name.find_last_of('.');
    return dot == std::string::npos ? name : name.substr(0, dot);
}

// A host buffer that is about to be overwritten whole (by a file or by a copy from the device): a std::vector would
// clear it first, one more pass over every byte of a tensor.
class HostBytes {
public:
    explicit HostBytes(size_t n) : p_(n ? new char[n] : nullptr), n_(n) {}
    char *data() { return p_.get(); }
    const char *data() const { return p_.get(); }
    size_t size() const { return n_; }
private:
    std::unique_ptr<char[]> p_;
    size_t n_;
};

inline HostBytes to_host(const Tensor &t) {
    HostBytes host((size_t)t.shape.bytes());
    dxh_check(dxh_memcpy_d2h(host.data(), t.data, host.size(), nullptr), "copy to host");
    return host;
}

// raw bytes to a file that is created or emptied first (stdutil/fs.cpp:18-29)
inline void write_exact(const std::string &path, const char *data, size_t bytes) {
    std::ofstream fs(path, std::ios::binary | std::ios::out | std::ios::trunc);
    if (!fs.is_open()) throw std::runtime_error("Failed to open file for writing: " + path);
    fs.write(data, (std::streamsize)bytes);
    if (!fs) throw std::runtime_error("Failed to write data to file: " + path);
}

inline void save_tensor(const Tensor &t, const std::string &path) {
    const std::string yaml = t.shape.to_yaml();
    write_exact(path + ".shape", yaml.data(), yaml.size());
    const size_t bytes = (size_t)t.shape.bytes();
    // A large tensor is copied from the device straight into the file's pages (a shared mapping of the file at its
    // final size) instead of into a buffer that is then written out: one pass over the bytes less (256 MiB: 40-95 ms
    // against 100-130; under 32 MiB the page faults of a fresh mapping cost more than the pass they save).
    if (bytes >= ((size_t)32 << 20)) {
        const std::string file = path + ".data";
        const int fd = ::open(file.c_str(), O_RDWR | O_CREAT | O_TRUNC, 0644);
        if (fd < 0) throw std::runtime_error("Failed to open file for writing: " + file);
        void *map = ::ftruncate(fd, (off_t)bytes) == 0 ? ::mmap(nullptr, bytes, PROT_READ | PROT_WRITE, MAP_SHARED, fd, 0) : MAP_FAILED;
        ::close(fd);
        if (map != MAP_FAILED) {
            const int rc = dxh_memcpy_d2h(map, t.data, bytes, nullptr);
            const bool unmapped = ::munmap(map, bytes) == 0;
            dxh_check(rc, "copy to host");
            if (!unmapped) throw std::runtime_error("Failed to write data to file: " + file);
            return;
        }
    }
    const HostBytes host = to_host(t);
    write_exact(path + ".data", host.data(), host.size());
}

// a file that must hold exactly `want` bytes (stdutil/fs.cpp:31-50)
inline HostBytes read_exact(const std::string &path, size_t want) {
    std::ifstream fs(path, std::ios::binary);
    if (!fs.is_open()) throw std::runtime_error("Failed to open file: " + path);
    fs.seekg(0, std::ios::end);
    size_t size = (size_t)fs.tellg();
    fs.seekg(0, std::ios::beg);
    if (size != want) throw std::runtime_error("file size mismatch: " + path);
    HostBytes buf(size);
    fs.read(buf.data(), (std::streamsize)size);
    if (fs.fail()) throw std::runtime_error("Failed to read file: " + path);
    return buf;
}

inline void load_tensor_data(const std::string &path, Tensor &t) {
    // accept both "<path>" and "<path>.data" like the two reference loaders do between them
    std::string file = path;
    if (file.size() < 5 || file.substr(file.size() - 5) != ".data") file += ".data";
    const size_t want = (size_t)t.shape.bytes();
    // A large file is copied to the device straight from its pages in the page cache (a private read-only mapping):
    // reading it into a buffer first is one more pass over every byte (256 MiB: 66 ms through a buffer, see below).
    // Same checks and messages as read_exact.
    if (want >= ((size_t)4 << 20)) {
        const int fd = ::open(file.c_str(), O_RDONLY);
        if (fd < 0) throw std::runtime_error("Failed to open file: " + file);
        struct stat st;
        if (::fstat(fd, &st) != 0 || (size_t)st.st_size != want) { ::close(fd); throw std::runtime_error("file size mismatch: " + file); }
        void *map = ::mmap(nullptr, want, PROT_READ, MAP_PRIVATE, fd, 0);
        ::close(fd);
        if (map != MAP_FAILED) {
            (void)::madvise(map, want, MADV_SEQUENTIAL);
            const int rc = dxh_memcpy_h2d(t.data, map, want, nullptr);
            ::munmap(map, want);
            dxh_check(rc, "copy to device");
            return;
        }
    }
    const HostBytes buf = read_exact(file, want);
    dxh_check(dxh_memcpy_h2d(t.data, buf.data(), buf.size(), nullptr), "copy to device");
}

inline std::pair<std::string, std::shared_ptr<Tensor>> load_tensor(const std::string &path) {
    std::ifstream fs(path + ".shape", std::ios::binary);
    if (!fs.is_open()) throw std::runtime_error("Failed to open shape file: " + path + ".shape");
    std::string text((std::istreambuf_iterator<char>(fs)), std::istreambuf_iterator<char>());
    Shape s = Shape::from_yaml(text);
    if (precision_bytes(s.dtype) == 0) throw std::runtime_error("unsupported dtype in " + path + ".shape");
    auto t = std::make_shared<Tensor>(s.shape, s.dtype);
    load_tensor_data(path, *t);
    // the reference takes the stem of the last path component ("a/b/w.x" -> "w"); a path without a
    // dot keeps its whole last component
    return {file_stem(path), t};
}

inline float half_bits_to_float(uint16_t h) {
    uint32_t s = uint32_t(h & 0x8000u) << 16, e = (h >> 10) & 0x1f, m = h & 0x3ff, u;
    if (e == 0) {
        if (m == 0) u = s;
        else { int sh = 0; while (!(m & 0x400)) { m <<= 1; ++sh; } u = s | ((113 - sh) << 23) | ((m & 0x3ff) << 13); }
    } else if (e == 31) u = s | 0x7f800000u | (m << 13);
    else u = s | ((e + 112) << 23) | (m << 13);
    float f;
    std::memcpy(&f, &u, 4);
    return f;
}

inline void print_element(std::ostream &os, const char *data, int64_t i, Precision p, const std::string &fmt) {
    char buf[128];
    switch (p) {
    case Precision::Float64: std::snprintf(buf, sizeof buf, fmt.c_str(), ((const double *)data)[i]); break;
    case Precision::Float32: std::snprintf(buf, sizeof buf, fmt.c_str(), (double)((const float *)data)[i]); break;
    case Precision::Float16: std::snprintf(buf, sizeof buf, fmt.c_str(), (double)half_bits_to_float(((const uint16_t *)data)[i])); break;
    case Precision::BFloat16: {
        uint32_t u = uint32_t(((const uint16_t *)data)[i]) << 16;
        float f;
        std::memcpy(&f, &u, 4);
        std::snprintf(buf, sizeof buf, fmt.c_str(), (double)f);
        break;
    }
    // integer formats reach here with their length modifier rewritten to "ll" (print_tensor)
    case Precision::Int64: std::snprintf(buf, sizeof buf, fmt.c_str(), (long long)((const int64_t *)data)[i]); break;
    case Precision::Int32: std::snprintf(buf, sizeof buf, fmt.c_str(), (long long)((const int32_t *)data)[i]); break;
    case Precision::Int16: std::snprintf(buf, sizeof buf, fmt.c_str(), (long long)((const int16_t *)data)[i]); break;
    case Precision::Int8: std::snprintf(buf, sizeof buf, fmt.c_str(), (long long)((const int8_t *)data)[i]); break;
    case Precision::Bool: std::snprintf(buf, sizeof buf, fmt.c_str(), (long long)((const uint8_t *)data)[i]); break;
    default: buf[0] = '?'; buf[1] = 0;
    }
    os << buf;
}

// The format of `print` arrives from the wire and goes to snprintf with one value: it must hold
// exactly one conversion, of the value's kind (floating: f e g a and capitals; integer: d i u x X o),
// with optional flags, width, precision and length modifier (not L: the value is a double); no %n,
// %s, %c, %p, no '*'.  "%%" is
// literal text.  (The reference passes the text through unchecked, stdutil/print.hpp.)
inline bool print_format_ok(const std::string &fmt, bool is_float) {
    int conversions = 0;
    for (size_t i = 0; i < fmt.size(); ++i) {
        if (fmt[i] != '%') continue;
        ++i;
        if (i < fmt.size() && fmt[i] == '%') continue;
        while (i < fmt.size() && std::strchr("-+ #0", fmt[i])) ++i;
        while (i < fmt.size() && std::isdigit((unsigned char)fmt[i])) ++i;
        if (i < fmt.size() && fmt[i] == '.') { ++i; while (i < fmt.size() && std::isdigit((unsigned char)fmt[i])) ++i; }
        while (i < fmt.size() && std::strchr(is_float ? "l" : "hljzt", fmt[i])) ++i;
        if (i >= fmt.size() || !std::strchr(is_float ? "fFeEgGaA" : "diuxXo", fmt[i])) return false;
        ++conversions;
    }
    return conversions == 1 && fmt.size() <= 64;
}

inline void print_tensor(const Tensor &t, std::string fmt, std::ostream &os) {
    const Precision p = t.shape.dtype;
    const bool is_float = (uint16_t(p) & uint16_t(Precision::Float)) != 0;
    if (fmt.empty()) fmt = is_float ? "%.4f" : "%d";
    if (!print_format_ok(fmt, is_float)) throw std::invalid_argument("print: format must hold one " + std::string(is_float ? "floating" : "integer") + " conversion: " + fmt);
    if (!is_float) {  // every integer value is passed as long long, whatever width the format named
        std::string ll;
        for (size_t i = 0; i < fmt.size(); ++i) {
            if (fmt[i] != '%') { ll += fmt[i]; continue; }
            ll += '%';
            if (i + 1 < fmt.size() && fmt[i + 1] == '%') { ll += '%'; ++i; continue; }
            for (++i; i < fmt.size() && !std::strchr("diuxXo", fmt[i]); ++i)
                if (!std::strchr("hljzt", fmt[i])) ll += fmt[i];
            ll += "ll";
            if (i < fmt.size()) ll += fmt[i];
        }
        fmt = ll;
    }
    const HostBytes host = to_host(t);
    const Shape &s = t.shape;
    os << "shape:[";
    for (int i = 0; i < s.dim(); ++i) os << s.shape[i] << (i + 1 < s.dim() ? ", " : "");
    os << "]" << std::endl;
    if (s.dim() == 1) {
        os << "[";
        for (int i = 0; i < s.shape[0]; ++i) { if (i) os << " "; print_element(os, host.data(), i, p, fmt); }
        os << "]" << std::endl;
        return;
    }
    const int rows = s.at(-2), cols = s.at(-1);
    const int64_t per = (int64_t)rows * cols;
    const int64_t mats = per > 0 ? s.size / per : 0;
    for (int64_t m = 0; m < mats; ++m) {
        // index of this matrix over the leading dims
        os << "[";
        int64_t rem = m;
        std::vector<int> idx(s.dim() - 2);
        for (int d = s.dim() - 3; d >= 0; --d) { idx[d] = (int)(rem % s.shape[d]); rem /= s.shape[d]; }
        for (size_t d = 0; d < idx.size(); ++d) os << idx[d] << (d + 1 < idx.size() ? ", " : "");
        os << "]=[" << std::endl;
        for (int i = 0; i < rows; ++i) {
            os << " [";
            for (int j = 0; j < cols; ++j) { if (j) os << " "; print_element(os, host.data(), (m * rows + i) * cols + j, p, fmt); }
            os << "]" << (i + 1 < rows ? "," : "") << std::endl;
        }
        os << "]" << std::endl;
    }
}

}  // namespace deepx
