// af<Op>(graph, {operands...}) with Op given as a class template: mode and element type are
// taken from the operands (same overload set as graphnn's include/nn/expr_sugar.h).
#ifndef EXPR_SUGAR_H
#define EXPR_SUGAR_H

#include "nn/factor_graph.h"

namespace gnn
{

#define GNN_AF_FOR(MODE, DTYPE)                                                                                \
    template<template <typename, typename> class FacType, typename... Args>                                   \
    typename FacType<MODE, DTYPE>::OutType af(FactorGraph& g,                                                 \
                                              std::vector< std::shared_ptr< TensorVar<MODE, DTYPE> > > op,    \
                                              Args&&... args)                                                  \
    {                                                                                                          \
        return af< FacType<MODE, DTYPE> >(g, op, std::forward<Args>(args)...);                                \
    }

GNN_AF_FOR(CPU, float)
GNN_AF_FOR(CPU, int)
GNN_AF_FOR(GPU, float)
GNN_AF_FOR(GPU, int)
#undef GNN_AF_FOR

}  // namespace gnn
#endif
