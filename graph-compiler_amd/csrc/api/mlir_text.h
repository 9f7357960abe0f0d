// Textual MLIR front end for the tensor-level modules the reference's tools take
// (gc-cpu-runner and benchgc's `--driver mlir`, test/benchgc/cases/*.mlir): one
// func.func over ranked tensors built from
//   tensor.empty, arith.constant (scalar or dense splat), linalg.fill,
//   linalg.matmul / matmul_transpose_a / matmul_transpose_b / batch_matmul /
//   batch_matmul_transpose_b,
//   linalg.matvec / vecmat / dot / batch_matvec / batch_vecmat / batch_reduce_matmul,
//   linalg.generic that is a contraction (multiply-accumulate over one reduction dim) or one point-wise op,
//   linalg.add / sub / mul / div / max / min / powf,
//   linalg.negf / exp / copy / abs / ceil / floor / erf / log / round / rsqrt / sqrt / square / tanh / reciprocal,
//   linalg.broadcast, linalg.transpose, linalg.softmax, linalg.reduce (sum),
//   tensor.collapse_shape / tensor.expand_shape, return,
//   and the reference's front-end dialect onednn_graph.{matmul, add, mul, sub, div, relu, sigmoid, pow, type_cast,
//   reduce_sum, reduce_mean} (test/mlir/test/gc/Dialect/OneDNNGraph/*.mlir).
// The first function of the text is compiled; anything after it is not looked at.
// The module becomes the same graph IR the JSON front end produces (graph.h), so
// verification, fusion and execution are shared.  Tensor ids: function argument
// i has id i; result j of the function has id (number of arguments) + j.
// Anything else in the module is reported as unsupported (std::logic_error ->
// dnnl_unimplemented); malformed text as std::invalid_argument.
#pragma once
#include "graph.h"

namespace gcapi {

Graph parse_mlir(const char *text);

} // namespace gcapi
