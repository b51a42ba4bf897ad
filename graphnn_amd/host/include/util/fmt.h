// Minimal fmt::sprintf: printf-style formatting into std::string.  graphnn vendors the
// cppformat library for the same call (include/util/fmt.h); the code that uses this API
// layer only needs sprintf with %s / %d / %f style arguments, std::string accepted for %s.
#ifndef GNN_FMT_H
#define GNN_FMT_H

#include <cstdio>
#include <string>
#include <vector>

namespace fmt
{
namespace detail
{
inline const char* printable(const std::string& s) { return s.c_str(); }
template<typename T> inline T printable(T v) { return v; }
}

template<typename... Args>
inline std::string sprintf(const char* format, Args&&... args)
{
    int need = std::snprintf(nullptr, 0, format, detail::printable(args)...);
    if (need <= 0) return std::string();
    std::vector<char> buf((size_t)need + 1);
    std::snprintf(buf.data(), buf.size(), format, detail::printable(args)...);
    return std::string(buf.data(), (size_t)need);
}

template<typename... Args>
inline std::string sprintf(const std::string& format, Args&&... args)
{
    return fmt::sprintf(format.c_str(), std::forward<Args>(args)...);
}
}

#endif
