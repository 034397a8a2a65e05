// String helpers used by the tensor descriptors and error messages.
// Same interface as the reference's src/utils/string_utils.h (fmtstr, vec2str, arr2str).
#pragma once
#include <cstdio>
#include <sstream>
#include <stdexcept>
#include <string>
#include <vector>

// printf-style formatting into a std::string.
template <typename... Args>
inline std::string fmtstr(const std::string& format, Args... args) {
    const int needed = std::snprintf(nullptr, 0, format.c_str(), args...);
    if (needed < 0) throw std::runtime_error("Error during formatting.");
    std::string out(static_cast<size_t>(needed) + 1, '\0');
    std::snprintf(&out[0], out.size(), format.c_str(), args...);
    out.resize(static_cast<size_t>(needed));
    return out;
}

// "(a, b, c)" from an iterator range.
template <typename It>
inline std::string isp_join_parenthesised(It first, It last) {
    std::ostringstream os;
    os << "(";
    for (It it = first; it != last; ++it) {
        if (it != first) os << ", ";
        os << *it;
    }
    os << ")";
    return os.str();
}

template <typename T>
inline std::string vec2str(std::vector<T> vec) {
    return isp_join_parenthesised(vec.begin(), vec.end());
}

template <typename T>
inline std::string arr2str(T* arr, size_t size) {
    return isp_join_parenthesised(arr, arr + size);
}
