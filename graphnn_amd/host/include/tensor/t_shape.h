// Shape of a tensor: dims plus the running products used for flat indexing
// (interface of graphnn's include/tensor/t_shape.h).
#ifndef T_SHAPE_H
#define T_SHAPE_H

#include "util/gnn_macros.h"
#include <string>
#include <vector>

namespace gnn
{

class TShape
{
public:
    TShape() {}
    TShape(std::vector<size_t> l) { Reshape(l); }

    void Reshape(std::vector<size_t> l)
    {
        dims = l;
        cnt.assign(dims.size(), 1);
        size_t run = 1;
        for (size_t i = dims.size(); i-- > 0;) {
            run *= dims[i];
            cnt[i] = run;              // cnt[i] = dims[i] * dims[i+1] * ...
        }
    }

    // number of elements from dimension `dim` on; an empty shape counts 0
    inline size_t Count(uint dim = 0)
    {
        if (dim == 0 && dims.empty()) return 0;
        ASSERT(dim < dims.size(), "dim is out of range");
        return cnt[dim];
    }

    size_t operator[](uint dim)
    {
        ASSERT(dim < dims.size(), "dim is out of range");
        return dims[dim];
    }

    size_t Coor2Idx(const std::vector<size_t>& l)
    {
        ASSERT(l.size() == dims.size(), "dimension mismatch");
        size_t idx = 0;
        for (size_t i = 0; i < l.size(); ++i) {
            ASSERT(l[i] < dims[i], "coordinate out of range");
            idx += l[i] * (i + 1 < dims.size() ? cnt[i + 1] : 1);
        }
        return idx;
    }

    std::string toString()
    {
        std::string s;
        for (size_t i = 0; i < dims.size(); ++i) s += (i ? " x " : "") + std::to_string(dims[i]);
        return s;
    }

    std::vector<size_t> dims;
    std::vector<size_t> cnt;
};

inline bool operator==(const TShape& a, const TShape& b) { return a.dims == b.dims; }
inline bool operator!=(const TShape& a, const TShape& b) { return !(a == b); }

}  // namespace gnn
#endif
