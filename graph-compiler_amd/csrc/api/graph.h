// Graph IR of a oneDNN-Graph partition: logical tensors, ops with attributes,
// input/output ids.  Built from the JSON schema the reference's parser accepts
// (src/dnnl/JsonParser.cpp:34-320 of the intel/graph-compiler tree) with the
// same error classes: std::invalid_argument -> dnnl_invalid_graph,
// std::logic_error -> dnnl_unimplemented.
#pragma once
#include <cstdint>
#include <map>
#include <string>
#include <unordered_map>
#include <utility>
#include <vector>

namespace gcapi {

enum class DT { undef, f16, bf16, f32, s32, s8, u8, f64, boolean, f8_e5m2, f8_e4m3, s4, u4 };
const char *dt_name(DT d);
int dt_size(DT d);      // bytes per element, 0 for sub-byte types
int dt_dnnl(DT d);      // dnnl_data_type_t value used across the kernel ABI (0 if none)

struct LTensor {
  size_t id = 0;
  DT dt = DT::undef;
  std::vector<int64_t> shape;
  bool unranked = false;
  bool strided = false;
  std::vector<int64_t> stride; // elements; only meaningful when strided
  bool constant = false;       // property_type == "constant"
  // set by the MLIR front end only:
  long alias_of = -1;          // id of the tensor whose storage this one shares (reshape views); same numel
  bool has_splat = false;      // every element equals `splat` (arith.constant dense<c>, linalg.fill of a constant)
  double splat = 0.0;
  int64_t numel() const {
    int64_t n = 1;
    for (auto d : shape)
      n *= d;
    return n;
  }
};

struct Attr {
  enum Type { Bool, S64, F32, S64Arr, F32Arr, Str } type = Bool;
  bool b = false;
  int64_t i = 0;
  float f = 0;
  std::vector<int64_t> ia;
  std::vector<float> fa;
  std::string s;
};

struct Op {
  std::string kind;
  std::map<std::string, Attr> attrs;
  std::vector<size_t> in, out;
  bool attr_bool(const char *k, bool dflt) const;
  int64_t attr_s64(const char *k, int64_t dflt) const;
  float attr_f32(const char *k, float dflt) const;
  std::string attr_str(const char *k, const char *dflt) const;
};

struct Graph {
  std::vector<Op> ops;
  std::unordered_map<size_t, LTensor> tensors;
  std::vector<size_t> input_ids;  // order of first use = argument order (JsonParser.cpp:183-199)
  std::vector<size_t> output_ids; // output_ports, or the last op's outputs (:91-94)
  // entries of a module's dlti.target_system_spec ("CPU" device: cache sizes, num_threads, max_vector_width, as
  // benchgc attaches them, test/benchgc/src/benchgc/mlir/util.py:187-197).  Read and reported; tiling on the GPU
  // follows the GPU's own parameters, so they steer nothing.
  std::vector<std::pair<std::string, int64_t>> target_hints;
};

// op kinds the reference front end accepts (src/dnnl/JsonParser.h:152-164) plus
// the extensions this library adds for the quantised MLP and attention paths
bool is_known_op(const std::string &kind);
bool is_extension_op(const std::string &kind);

Graph parse_graph(const char *json);

// ops only the MLIR front end produces (mlir_text.h): Maximum, Minimum, Exp, Neg, Abs, Ceil, Floor, Erf, Log, Round,
// Rsqrt, Sqrt, Square, Tanh, Reciprocal (element-wise), Reshape (a view),
// Transpose {perm}, BroadcastTo {dims: the result dimensions that are added}
bool is_internal_op(const std::string &kind);

// Checks every op's operand/result shapes and dtypes (the role of the MLIR op
// verifiers, include/gc/Dialect/OneDNNGraph/OneDNNGraphOps.td and
// lib/gc/Dialect/OneDNNGraph/OneDNNGraphOps.cpp:204-310).  Throws
// std::runtime_error, which the C API reports as dnnl_runtime_error like a
// failed JitModule::create.
void verify_graph(const Graph &g);

// numpy-style broadcast of two shapes; false when incompatible
bool broadcast_shape(const std::vector<int64_t> &a, const std::vector<int64_t> &b, std::vector<int64_t> &out);
// canonical (non-negative, sorted, unique) reduce axes; empty input = all axes
std::vector<int64_t> canonical_axes(const std::vector<int64_t> &axes, int64_t rank);

} // namespace gcapi
