// Everything of the tensor layer (same entry header as graphnn's include/tensor/tensor_all.h).
#ifndef TENSOR_ALL_H
#define TENSOR_ALL_H

#include "tensor/tensor.h"
#include "tensor/cpu_dense_tensor.h"
#include "tensor/cpu_sparse_tensor.h"
#include "tensor/cpu_row_sparse_tensor.h"
#include "tensor/gpu_handle.h"
#include "tensor/gpu_dense_tensor.h"
#include "tensor/gpu_sparse_tensor.h"
#include "tensor/gpu_row_sparse_tensor.h"

#endif
