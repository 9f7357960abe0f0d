#include "graph.h"

#include <algorithm>
#include <limits>
#include <set>
#include <stdexcept>

#include "json.h"

namespace gcapi {

const char *dt_name(DT d) {
  static const char *n[] = {"undef", "f16", "bf16", "f32", "s32", "s8", "u8", "f64", "boolean", "f8_e5m2", "f8_e4m3", "s4", "u4"};
  return n[(int)d];
}
int dt_size(DT d) {
  switch (d) {
  case DT::f16: case DT::bf16: return 2;
  case DT::f32: case DT::s32: return 4;
  case DT::s8: case DT::u8: case DT::boolean: case DT::f8_e5m2: case DT::f8_e4m3: return 1;
  case DT::f64: return 8;
  default: return 0;
  }
}
int dt_dnnl(DT d) {
  switch (d) {
  case DT::f16: return 1;
  case DT::bf16: return 2;
  case DT::f32: return 3;
  case DT::s32: return 4;
  case DT::s8: return 5;
  case DT::u8: return 6;
  default: return 0;
  }
}

bool Op::attr_bool(const char *k, bool dflt) const {
  auto it = attrs.find(k);
  if (it == attrs.end())
    return dflt;
  if (it->second.type == Attr::Bool)
    return it->second.b;
  if (it->second.type == Attr::S64)
    return it->second.i != 0;
  throw std::invalid_argument(std::string("Invalid attribute type: ") + k);
}
int64_t Op::attr_s64(const char *k, int64_t dflt) const {
  auto it = attrs.find(k);
  if (it == attrs.end())
    return dflt;
  if (it->second.type != Attr::S64)
    throw std::invalid_argument(std::string("Invalid attribute type: ") + k);
  return it->second.i;
}
float Op::attr_f32(const char *k, float dflt) const {
  auto it = attrs.find(k);
  if (it == attrs.end())
    return dflt;
  if (it->second.type == Attr::F32)
    return it->second.f;
  if (it->second.type == Attr::S64)
    return (float)it->second.i;
  throw std::invalid_argument(std::string("Invalid attribute type: ") + k);
}
std::string Op::attr_str(const char *k, const char *dflt) const {
  auto it = attrs.find(k);
  if (it == attrs.end())
    return dflt;
  if (it->second.type != Attr::Str)
    throw std::invalid_argument(std::string("Invalid attribute type: ") + k);
  return it->second.s;
}

static const std::set<std::string> &reference_ops() {
  static const std::set<std::string> s = {"Add", "Divide", "MatMul", "Multiply", "Pow", "ReduceMean", "ReduceSum",
                                          "ReLU", "Sigmoid", "Subtract", "Typecast"};
  return s;
}
static const std::set<std::string> &extension_ops() {
  // spelled as in the oneDNN Graph specification; semantics from the reference's
  // legacy core (GELU, Dequantize, Quantize, SoftMax) -- see the README
  // and the element-wise ops of that specification the point-wise kernels have anyway
  static const std::set<std::string> s = {"GELU", "Dequantize", "Quantize", "SoftMax",    "TypeCast", "Abs",    "Exp", "Log",
                                          "Maximum", "Minimum", "Reciprocal", "Sqrt", "Square", "Tanh"};
  return s;
}
bool is_known_op(const std::string &k) { return reference_ops().count(k) || extension_ops().count(k); }
bool is_extension_op(const std::string &k) { return extension_ops().count(k) != 0; }
bool is_internal_op(const std::string &k) {
  static const std::set<std::string> s = {"Maximum", "Minimum", "Exp",  "Neg",    "Abs",  "Ceil",       "Floor",   "Erf",       "Log",
                                          "Round",   "Rsqrt",   "Sqrt", "Square", "Tanh", "Reciprocal", "Reshape", "Transpose", "BroadcastTo"};
  return s.count(k) != 0;
}

namespace {

[[noreturn]] void bad(const std::string &m) { throw std::invalid_argument(m); }
[[noreturn]] void unimpl(const std::string &m) { throw std::logic_error(m); }

const std::string &want_str(const JValue &v, const char *what) {
  if (v.type != JValue::Str)
    bad(std::string("String expected: ") + what);
  return v.str;
}
int64_t want_int(const JValue &v, const char *what) {
  if (v.type == JValue::Bool)
    return v.b ? 1 : 0;
  if (v.type != JValue::Num)
    bad(std::string("Number expected: ") + what);
  return v.inum;
}
std::vector<int64_t> want_int_array(const JValue &v, const char *what) {
  if (v.type != JValue::Arr)
    bad(std::string("Array expected: ") + what);
  std::vector<int64_t> o;
  for (auto &e : v.arr)
    o.push_back(want_int(e, what));
  return o;
}

DT parse_dtype(const std::string &s) {
  static const std::map<std::string, DT> m = {
      {"f16", DT::f16}, {"bf16", DT::bf16}, {"f32", DT::f32}, {"s32", DT::s32}, {"s8", DT::s8}, {"u8", DT::u8},
      {"f64", DT::f64}, {"boolean", DT::boolean}, {"f8_e5m2", DT::f8_e5m2}, {"f8_e4m3", DT::f8_e4m3},
      {"s4", DT::s4}, {"u4", DT::u4}};
  auto it = m.find(s);
  if (it == m.end())
    unimpl("Unsupported dtype: " + s); // JsonParser.cpp:277-280
  return it->second;
}

// JsonParser.cpp:267-320
LTensor read_tensor(const JValue &v) {
  if (v.type != JValue::Obj)
    bad("Tensor object expected");
  LTensor t;
  bool has_dtype = false, has_id = false;
  for (auto &kv : v.obj) {
    const std::string &k = kv.first;
    if (k == "id") {
      t.id = (size_t)want_int(kv.second, "id");
      has_id = true;
    } else if (k == "dtype") {
      t.dt = parse_dtype(want_str(kv.second, "dtype"));
      has_dtype = true;
    } else if (k == "shape") {
      t.shape = want_int_array(kv.second, "shape");
    } else if (k == "stride") {
      t.stride = want_int_array(kv.second, "stride");
    } else if (k == "layout_type") {
      const std::string &s = want_str(kv.second, "layout_type");
      if (s == "strided")
        t.strided = true;
      else if (s != "undef" && s != "any")
        unimpl("Unsupported layout_type: " + s);
    } else if (k == "property_type") {
      const std::string &s = want_str(kv.second, "property_type");
      if (s == "constant")
        t.constant = true;
      else if (s != "undef" && s != "variable")
        unimpl("Unsupported property_type: " + s);
    } else {
      bad("Unrecognized key: " + k);
    }
  }
  if (!has_dtype)
    bad("dtype is not specified");
  if (!has_id)
    bad("tensor id is not specified");
  if (t.shape.size() == 1 && t.shape[0] == std::numeric_limits<int64_t>::min()) {
    t.unranked = true;
    t.shape.clear();
  }
  if (!t.strided)
    t.stride.clear();
  else if (t.stride.size() != t.shape.size())
    bad("stride rank differs from shape rank for tensor " + std::to_string(t.id));
  return t;
}

// JsonParser.cpp:228-265
Attr read_attr(const JValue &v, const std::string &name) {
  if (v.type != JValue::Obj || v.obj.size() < 2 || v.obj[0].first != "type")
    bad("Key expected: type");
  if (v.obj[1].first != "value")
    bad("Unrecognized key: " + v.obj[1].first);
  if (v.obj.size() > 2)
    bad("Unrecognized key: " + v.obj[2].first);
  const std::string &ty = want_str(v.obj[0].second, "type");
  const JValue &val = v.obj[1].second;
  Attr a;
  if (ty == "bool") {
    a.type = Attr::Bool;
    a.b = want_int(val, name.c_str()) != 0;
  } else if (ty == "s64") {
    a.type = Attr::S64;
    a.i = want_int(val, name.c_str());
  } else if (ty == "f32") {
    a.type = Attr::F32;
    if (val.type != JValue::Num)
      bad("Number expected: " + name);
    a.f = (float)val.num;
  } else if (ty == "s64[]") {
    a.type = Attr::S64Arr;
    a.ia = want_int_array(val, name.c_str());
  } else if (ty == "f32[]") {
    a.type = Attr::F32Arr;
    if (val.type != JValue::Arr)
      bad("Array expected: " + name);
    for (auto &e : val.arr) {
      if (e.type != JValue::Num)
        bad("Number expected: " + name);
      a.fa.push_back((float)e.num);
    }
  } else if (ty == "string") {
    a.type = Attr::Str;
    a.s = want_str(val, name.c_str());
  } else {
    unimpl("Unsupported attribute type: " + ty);
  }
  return a;
}

} // namespace

// JsonParser.cpp:34-133 (top level) and :135-226 (one op)
Graph parse_graph(const char *json) {
  if (!json)
    bad("null graph");
  JValue root = parse_json(json);
  if (root.type != JValue::Obj)
    bad("Object expected");
  Graph g;
  std::vector<size_t> input_ports;
  bool has_in_ports = false, has_out_ports = false;
  std::set<size_t> produced;
  std::vector<size_t> last_outputs;

  for (auto &kv : root.obj) {
    const std::string &k = kv.first;
    if (k == "version") {
      want_str(kv.second, "version");
    } else if (k == "engine_kind") {
      const std::string &s = want_str(kv.second, "engine_kind");
      // the reference accepts "cpu" only; "gpu" is accepted too since that is
      // where this library runs.  Reference JSONs run unchanged.
      if (s != "cpu" && s != "gpu")
        unimpl("Unsupported engine: " + s);
    } else if (k == "fpmath_mode") {
      const std::string &s = want_str(kv.second, "fpmath_mode");
      if (s != "strict" && s != "any")
        unimpl("Unsupported fpmath_mode: " + s + ". Only 'strict' and 'any' are currently supported.");
    } else if (k == "input_ports") {
      has_in_ports = true;
      for (auto v : want_int_array(kv.second, "input_ports"))
        input_ports.push_back((size_t)v);
    } else if (k == "output_ports") {
      has_out_ports = true;
      for (auto v : want_int_array(kv.second, "output_ports"))
        g.output_ids.push_back((size_t)v);
    } else if (k == "graph") {
      if (kv.second.type != JValue::Arr)
        bad("Array expected: graph");
      for (auto &jop : kv.second.arr) {
        if (jop.type != JValue::Obj)
          bad("Operation object expected");
        Op op;
        bool has_kind = false;
        for (auto &okv : jop.obj) {
          const std::string &ok = okv.first;
          if (ok == "id") {
            want_int(okv.second, "id");
          } else if (ok == "name") {
            want_str(okv.second, "name");
          } else if (ok == "kind") {
            op.kind = want_str(okv.second, "kind");
            if (!is_known_op(op.kind))
              unimpl("Unsupported operation: " + op.kind);
            has_kind = true;
          } else if (ok == "attrs") {
            if (okv.second.type != JValue::Obj)
              bad("Object expected: attrs");
            for (auto &akv : okv.second.obj) {
              Attr a = read_attr(akv.second, akv.first);
              if (akv.first == "auto_broadcast") { // string -> bool, JsonParser.cpp:164-177
                if (a.type != Attr::Str)
                  bad("Invalid attribute type: auto_broadcast");
                if (a.s != "numpy" && a.s != "none")
                  bad("Invalid auto_broadcast attribute value: " + a.s);
                Attr b;
                b.type = Attr::Bool;
                b.b = a.s == "numpy";
                a = b;
              }
              op.attrs[akv.first] = a;
            }
          } else if (ok == "inputs") {
            if (okv.second.type != JValue::Arr)
              bad("Array expected: inputs");
            for (auto &jt : okv.second.arr) {
              LTensor t = read_tensor(jt);
              auto it = g.tensors.find(t.id);
              if (it == g.tensors.end()) {
                g.tensors[t.id] = t; // unseen id: a function argument
                g.input_ids.push_back(t.id);
              } else if (it->second.dt != t.dt || it->second.shape != t.shape || it->second.unranked != t.unranked) {
                bad("Type mismatch for input: " + std::to_string(t.id));
              }
              op.in.push_back(t.id);
            }
          } else if (ok == "outputs") {
            if (okv.second.type != JValue::Arr)
              bad("Array expected: outputs");
            for (auto &jt : okv.second.arr) {
              LTensor t = read_tensor(jt);
              op.out.push_back(t.id);
              // registered after the whole op is read (inputs may follow outputs in the text)
              if (produced.count(t.id) || g.tensors.count(t.id))
                bad("Duplicate output id: " + std::to_string(t.id));
              produced.insert(t.id);
              g.tensors[t.id] = t;
            }
          } else {
            bad("Unrecognized key: " + ok);
          }
        }
        if (!has_kind)
          bad("Operation kind is not specified");
        last_outputs = op.out;
        g.ops.push_back(std::move(op));
      }
    } else {
      bad("Unrecognized key: " + k);
    }
  }

  if (has_in_ports) {
    if (input_ports.size() != g.input_ids.size())
      bad("Length mismatch between input_ports and inputs: " + std::to_string(g.input_ids.size()));
    for (auto id : g.input_ids)
      if (std::find(input_ports.begin(), input_ports.end(), id) == input_ports.end())
        bad("Input not found in input_ports: " + std::to_string(id));
  }
  if (!has_out_ports)
    g.output_ids = last_outputs;
  for (auto id : g.output_ids)
    if (!g.tensors.count(id))
      bad("Output value not found: " + std::to_string(id));
  return g;
}

bool broadcast_shape(const std::vector<int64_t> &a, const std::vector<int64_t> &b, std::vector<int64_t> &out) {
  size_t r = std::max(a.size(), b.size());
  out.assign(r, 1);
  for (size_t i = 0; i < r; i++) {
    int64_t da = i < r - a.size() ? 1 : a[i - (r - a.size())];
    int64_t db = i < r - b.size() ? 1 : b[i - (r - b.size())];
    if (da != db && da != 1 && db != 1)
      return false;
    out[i] = da == 1 ? db : da;
  }
  return true;
}

std::vector<int64_t> canonical_axes(const std::vector<int64_t> &axes, int64_t rank) {
  // no axes: nothing is reduced, the op returns its operand
  // (lib/gc/Dialect/OneDNNGraph/OneDNNGraphOps.cpp:116-120, lib/gc/Transforms/OneDNNGraphToLinalg.cpp:320-324)
  std::vector<int64_t> o;
  for (auto a : axes)
    o.push_back(a < 0 ? a + rank : a);
  std::sort(o.begin(), o.end());
  o.erase(std::unique(o.begin(), o.end()), o.end());
  return o;
}

namespace {
[[noreturn]] void vfail(const Op &op, const std::string &m) { throw std::runtime_error("verify " + op.kind + ": " + m); }
bool is_float(DT d) { return d == DT::f32 || d == DT::bf16 || d == DT::f16; }
} // namespace

void verify_graph(const Graph &g) {
  for (auto &op : g.ops) {
    auto T = [&](size_t id) -> const LTensor & { return g.tensors.at(id); };
    for (auto id : op.in)
      if (T(id).unranked)
        vfail(op, "unranked operand");
    for (auto id : op.out)
      if (T(id).unranked)
        vfail(op, "unranked result");
    const std::string &k = op.kind;
    if (k == "Add" || k == "Subtract" || k == "Multiply" || k == "Divide" || k == "Maximum" || k == "Minimum") {
      if (op.in.size() != 2 || op.out.size() != 1)
        vfail(op, "expects 2 operands and 1 result");
      std::vector<int64_t> o;
      if (!is_float(T(op.in[0]).dt) || !is_float(T(op.in[1]).dt))
        vfail(op, "float tensors only");
      if (!broadcast_shape(T(op.in[0]).shape, T(op.in[1]).shape, o) || o != T(op.out[0]).shape)
        vfail(op, "operand shapes do not broadcast to the result shape");
      if (!op.attr_bool("auto_broadcast", true) && T(op.in[0]).shape != T(op.in[1]).shape)
        vfail(op, "auto_broadcast is none but shapes differ");
    } else if (k == "ReLU" || k == "Sigmoid" || k == "Pow" || k == "GELU" || k == "Exp" || k == "Neg" || k == "Abs" ||
               k == "Ceil" || k == "Floor" || k == "Erf" || k == "Log" || k == "Round" || k == "Rsqrt" || k == "Sqrt" ||
               k == "Square" || k == "Tanh" || k == "Reciprocal") {
      if (op.in.size() != 1 || op.out.size() != 1)
        vfail(op, "expects 1 operand and 1 result");
      if (T(op.in[0]).shape != T(op.out[0]).shape || T(op.in[0]).dt != T(op.out[0]).dt || !is_float(T(op.in[0]).dt))
        vfail(op, "operand and result types differ");
      if (k == "Pow" && !op.attrs.count("beta"))
        vfail(op, "attribute beta is required");
    } else if (k == "Reshape") {
      if (op.in.size() != 1 || op.out.size() != 1 || T(op.in[0]).numel() != T(op.out[0]).numel() ||
          T(op.in[0]).dt != T(op.out[0]).dt)
        vfail(op, "a reshape keeps the element count and type");
    } else if (k == "Transpose") {
      const auto &in = T(op.in[0]), &out = T(op.out[0]);
      auto it = op.attrs.find("perm");
      if (op.in.size() != 1 || op.out.size() != 1 || it == op.attrs.end() || it->second.ia.size() != in.shape.size() ||
          out.shape.size() != in.shape.size() || in.dt != out.dt)
        vfail(op, "permutation does not fit the operand");
      std::vector<char> seen(in.shape.size(), 0);
      for (size_t d = 0; d < in.shape.size(); d++) {
        int64_t q = it->second.ia[d];
        if (q < 0 || q >= (int64_t)in.shape.size() || seen[(size_t)q] || out.shape[d] != in.shape[(size_t)q])
          vfail(op, "permutation does not fit the operand");
        seen[(size_t)q] = 1;
      }
    } else if (k == "BroadcastTo") {
      const auto &in = T(op.in[0]), &out = T(op.out[0]);
      auto it = op.attrs.find("dims");
      if (op.in.size() != 1 || op.out.size() != 1 || it == op.attrs.end() || in.dt != out.dt ||
          in.shape.size() + it->second.ia.size() != out.shape.size())
        vfail(op, "broadcast dimensions do not fit");
      size_t src = 0;
      for (size_t d = 0; d < out.shape.size(); d++) {
        bool added = std::find(it->second.ia.begin(), it->second.ia.end(), (int64_t)d) != it->second.ia.end();
        if (!added && (src >= in.shape.size() || in.shape[src++] != out.shape[d]))
          vfail(op, "broadcast dimensions do not fit");
      }
    } else if (k == "Typecast" || k == "TypeCast") {
      if (op.in.size() != 1 || op.out.size() != 1 || T(op.in[0]).shape != T(op.out[0]).shape)
        vfail(op, "operand and result shapes differ");
      if (!is_float(T(op.in[0]).dt) || !is_float(T(op.out[0]).dt))
        vfail(op, "float tensors only");
    } else if (k == "ReduceSum" || k == "ReduceMean") {
      if (op.in.size() != 1 || op.out.size() != 1)
        vfail(op, "expects 1 operand and 1 result");
      const auto &in = T(op.in[0]);
      int64_t rank = (int64_t)in.shape.size();
      std::vector<int64_t> axes;
      auto it = op.attrs.find("axes");
      if (it != op.attrs.end())
        axes = it->second.ia;
      for (auto a : axes)
        if (a >= rank || a < -rank)
          vfail(op, "Reduce axis not valid!");
      auto ca = canonical_axes(axes, rank);
      bool keep = op.attr_bool("keep_dims", false);
      std::vector<int64_t> o;
      for (int64_t d = 0; d < rank; d++) {
        bool red = std::find(ca.begin(), ca.end(), d) != ca.end();
        if (!red)
          o.push_back(in.shape[d]);
        else if (keep)
          o.push_back(1);
      }
      if (o != T(op.out[0]).shape || in.dt != T(op.out[0]).dt)
        vfail(op, "result type does not match the reduced operand");
    } else if (k == "MatMul") {
      if (op.in.size() < 2 || op.in.size() > 3 || op.out.size() != 1)
        vfail(op, "expects 2 or 3 operands and 1 result");
      const auto &a = T(op.in[0]), &b = T(op.in[1]);
      bool ta = op.attr_bool("transpose_a", false), tb = op.attr_bool("transpose_b", false);
      size_t ra = a.shape.size(), rb = b.shape.size();
      std::vector<int64_t> o;
      auto rowcol = [](const LTensor &t, bool tr) {
        size_t r = t.shape.size();
        return tr ? std::make_pair(t.shape[r - 1], t.shape[r - 2]) : std::make_pair(t.shape[r - 2], t.shape[r - 1]);
      };
      if (ra == 0 || rb == 0)
        vfail(op, "rank-0 operand");
      if (ra == 1 && rb == 1) {
        if (a.shape[0] != b.shape[0])
          vfail(op, "contraction sizes differ");
        o.push_back(1);
      } else if (ra == 1) {
        auto rc = rowcol(b, tb);
        if (a.shape[0] != rc.first)
          vfail(op, "contraction sizes differ");
        o.assign(b.shape.begin(), b.shape.end() - 2);
        o.push_back(rc.second);
      } else if (rb == 1) {
        auto rc = rowcol(a, ta);
        if (rc.second != b.shape[0])
          vfail(op, "contraction sizes differ");
        o.assign(a.shape.begin(), a.shape.end() - 2);
        o.push_back(rc.first);
      } else {
        std::vector<int64_t> ba(a.shape.begin(), a.shape.end() - 2), bb(b.shape.begin(), b.shape.end() - 2);
        if (!broadcast_shape(ba, bb, o))
          vfail(op, "batch dimensions do not broadcast");
        auto l = rowcol(a, ta), r = rowcol(b, tb);
        if (l.second != r.first)
          vfail(op, "contraction sizes differ");
        o.push_back(l.first);
        o.push_back(r.second);
      }
      if (o != T(op.out[0]).shape)
        vfail(op, "result shape does not match the operands");
      if (op.in.size() == 3) {
        const auto &bias = T(op.in[2]);
        std::vector<int64_t> tmp;
        if (!(bias.shape.size() == 1 || bias.shape.size() == o.size()) || !broadcast_shape(o, bias.shape, tmp) ||
            tmp != o)
          vfail(op, "bias does not broadcast to the result");
      }
      if (!is_float(a.dt) || a.dt != b.dt)
        vfail(op, "operand element types differ");
      // same element type, or (extension) 16-bit operands with an f32 result
      if (T(op.out[0]).dt != a.dt && !(T(op.out[0]).dt == DT::f32 && a.dt == DT::bf16))
        vfail(op, "result element type differs from the operands");
    } else if (k == "SoftMax") {
      if (op.in.size() != 1 || op.out.size() != 1 || T(op.in[0]).shape != T(op.out[0]).shape)
        vfail(op, "operand and result shapes differ");
      int64_t rank = (int64_t)T(op.in[0]).shape.size(), ax = op.attr_s64("axis", 1);
      if (ax >= rank || ax < -rank)
        vfail(op, "axis out of range");
    } else if (k == "Dequantize" || k == "Quantize") {
      if (op.in.size() != 1 || op.out.size() != 1 || T(op.in[0]).shape != T(op.out[0]).shape)
        vfail(op, "operand and result shapes differ");
      auto sc = op.attrs.find("scales");
      if (sc == op.attrs.end() || sc->second.type != Attr::F32Arr || sc->second.fa.empty())
        vfail(op, "attribute scales (f32[]) is required");
      const LTensor &q = k == "Dequantize" ? T(op.in[0]) : T(op.out[0]);
      const LTensor &f = k == "Dequantize" ? T(op.out[0]) : T(op.in[0]);
      if (!(q.dt == DT::u8 || q.dt == DT::s8) || !is_float(f.dt))
        vfail(op, "expects an 8-bit integer tensor on the quantised side and a float tensor on the other");
      int64_t rank = (int64_t)q.shape.size(), ax = op.attr_s64("axis", 1);
      size_t ns = sc->second.fa.size();
      if (ns > 1) {
        if (ax >= rank || ax < -rank)
          vfail(op, "axis out of range");
        if ((int64_t)ns != q.shape[ax < 0 ? ax + rank : ax])
          vfail(op, "number of scales differs from the channel dimension");
      }
      auto zp = op.attrs.find("zps");
      if (zp != op.attrs.end() && zp->second.ia.size() != 1 && zp->second.ia.size() != ns)
        vfail(op, "number of zero points differs from the number of scales");
    }
  }
}

} // namespace gcapi
