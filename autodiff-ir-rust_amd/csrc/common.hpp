// Shared small utilities: error type, string formatting, shape helpers.
#pragma once
#include <cstdarg>
#include <cstdint>
#include <cstdio>
#include <stdexcept>
#include <string>
#include <vector>

namespace adhip {

using Shape = std::vector<int64_t>;

struct Error : std::runtime_error {
    using std::runtime_error::runtime_error;
};

inline std::string strf(const char* fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    va_list ap2;
    va_copy(ap2, ap);
    int n = vsnprintf(nullptr, 0, fmt, ap);
    va_end(ap);
    std::string s((size_t)(n > 0 ? n : 0), '\0');
    if (n > 0) vsnprintf(&s[0], (size_t)n + 1, fmt, ap2);
    va_end(ap2);
    return s;
}

#define ADHIP_CHECK(cond, ...)                                   \
    do {                                                         \
        if (!(cond)) throw ::adhip::Error(::adhip::strf(__VA_ARGS__)); \
    } while (0)

// Product of the dims; sizes come from the caller's command stream, so a product that does not fit is an error of
// the program, not undefined behaviour here.
inline int64_t numel(const Shape& s) {
    int64_t n = 1;
    for (auto d : s)
        if (__builtin_mul_overflow(n, d, &n)) throw ::adhip::Error("tensor size overflows 64 bits");
    return n;
}

inline Shape row_major_strides(const Shape& s) {
    Shape r(s.size(), 1);
    for (int i = (int)s.size() - 2; i >= 0; --i) r[i] = r[i + 1] * s[i + 1];
    return r;
}

inline std::string shape_str(const Shape& s) {
    std::string o = "[";
    for (size_t i = 0; i < s.size(); ++i) o += (i ? "," : "") + std::to_string(s[i]);
    return o + "]";
}

}  // namespace adhip
