// Everything of the operator layer that the structure2vec path uses
// (same entry header as graphnn's include/nn/nn_all.h).
#ifndef NN_ALL_H
#define NN_ALL_H

#include "nn/variable.h"
#include "nn/factor.h"
#include "nn/factor_graph.h"
#include "nn/expr_sugar.h"
#include "nn/msg_pass.h"
#include "nn/matmul.h"
#include "nn/relu.h"
#include "nn/elewise_add.h"
#include "nn/cross_entropy.h"
#include "nn/reduce_mean.h"
#include "nn/arg_max.h"
#include "nn/in_top_k.h"
#include "nn/type_cast.h"
#include "nn/softmax.h"
#include "nn/jagged_softmax.h"
#include "nn/reduce.h"
#include "nn/fully_connected.h"
#include "nn/param_set.h"
#include "nn/optimizer.h"

#endif
