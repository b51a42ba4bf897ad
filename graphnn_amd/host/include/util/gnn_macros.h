// Host-side API layer over libgnnhip: enums, type tags and the assertion macro.
// Names and values follow graphnn's include/util/gnn_macros.h so code written
// against graphnn (its graph_classification example in particular) compiles
// unchanged; the implementation underneath is this repository's.
#ifndef GNN_MACROS_H
#define GNN_MACROS_H

#include <cstddef>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <exception>
#include <iostream>
#include <stdexcept>
#include <string>
#include <execinfo.h>
#include <unistd.h>

namespace gnn
{

typedef unsigned int uint;

enum class MatType { dense, sparse, row_sparse };
enum class PropErr { N = 0, T = 1 };
enum class Trans { N = 0, T = 1 };
enum class MatMode { cpu = 0, gpu = 1 };
enum class Phase { TRAIN = 0, TEST = 1 };
enum class EleType { FLOAT32 = 0, FLOAT64 = 1, INT32 = 2, UNKNOWN = 3 };

template<typename Dtype> inline EleType Dtype2Enum();
template<> inline EleType Dtype2Enum<float>() { return EleType::FLOAT32; }
template<> inline EleType Dtype2Enum<double>() { return EleType::FLOAT64; }
template<> inline EleType Dtype2Enum<int>() { return EleType::INT32; }

// template tags: where a tensor lives and how it is stored
struct CPU { static const MatMode type = MatMode::cpu; };
struct GPU { static const MatMode type = MatMode::gpu; };
struct DENSE { static const MatType type = MatType::dense; };
struct CSR_SPARSE { static const MatType type = MatType::sparse; };
struct ROW_SPARSE { static const MatType type = MatType::row_sparse; };

// graphnn's failure convention: print the condition, a short backtrace, terminate.
inline void gnn_assert_fail(const char* cond, const char* file, int line, const std::string& msg)
{
    std::cerr << "Assertion `" << cond << "` failed in " << file << " line " << line << ": " << msg << std::endl;
    void* frames[10];
    int depth = backtrace(frames, 10);
    backtrace_symbols_fd(frames, depth, STDERR_FILENO);
    std::terminate();
}

}  // namespace gnn

#include <sstream>
#define ASSERT(condition, message)                                                          \
    do {                                                                                    \
        if (!(condition)) {                                                                 \
            std::ostringstream gnn_assert_os__;                                             \
            gnn_assert_os__ << message;                                                     \
            ::gnn::gnn_assert_fail(#condition, __FILE__, __LINE__, gnn_assert_os__.str());  \
        }                                                                                   \
    } while (false)

#define NOT_IMPLEMENTED { throw std::logic_error(std::string("not implemented virtual func: ") + std::string(__FUNCTION__)); }

// dispatch on the storage kind of a tensor variable
#define MAT_TYPE_SWITCH(type, matType, ...)                         \
    switch (type) {                                                 \
    case ::gnn::MatType::dense: { typedef ::gnn::DENSE matType; {__VA_ARGS__} } break;        \
    case ::gnn::MatType::sparse: { typedef ::gnn::CSR_SPARSE matType; {__VA_ARGS__} } break;  \
    default: throw std::logic_error("unknown type");                \
    }

#endif
