// Umbrella header of the DIA product path.
#ifndef __CUV_DIA_ALL_HPP__
#define __CUV_DIA_ALL_HPP__
#include <cuv/basics/dia_matrix.hpp>
#include <cuv/basics/filter_factory.hpp>
#include <cuv/basics/tensor.hpp>
#include <cuv/convert/convert.hpp>
#include <cuv/matrix_ops/densedense_to_sparse.hpp>
#include <cuv/matrix_ops/diagonals.hpp>
#include <cuv/matrix_ops/host_ops.hpp>
#include <cuv/matrix_ops/matrix_ops.hpp>
#include <cuv/tensor_ops/rprop.hpp>
#include <cuv/tensor_ops/tensor_ops.hpp>
#include <cuv/tools/cuv_general.hpp>
#endif
