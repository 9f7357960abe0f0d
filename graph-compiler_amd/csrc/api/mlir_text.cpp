#include "mlir_text.h"

#include <algorithm>
#include <cctype>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <map>
#include <set>
#include <stdexcept>

namespace gcapi {
namespace {

[[noreturn]] void bad(const std::string &m) { throw std::invalid_argument("MLIR: " + m); }
[[noreturn]] void unimpl(const std::string &m) { throw std::logic_error("MLIR: " + m); }

struct Type {
  bool tensor = false;
  DT dt = DT::undef;
  std::vector<int64_t> shape;
};

DT elem_type(const std::string &s) {
  if (s == "f32")
    return DT::f32;
  if (s == "bf16")
    return DT::bf16;
  if (s == "f16")
    return DT::f16;
  if (s == "f64")
    return DT::f64;
  if (s == "i32" || s == "si32")
    return DT::s32;
  if (s == "i8" || s == "si8")
    return DT::s8;
  if (s == "ui8")
    return DT::u8;
  if (s == "i1")
    return DT::boolean;
  unimpl("element type " + s);
}

// A cursor over the module text.  Whitespace and // comments separate tokens.
struct Cursor {
  const char *p, *end;
  explicit Cursor(const char *t) : p(t), end(t + strlen(t)) {}
  void ws() {
    for (;;) {
      while (p < end && isspace((unsigned char)*p))
        p++;
      if (p + 1 < end && p[0] == '/' && p[1] == '/') {
        while (p < end && *p != '\n')
          p++;
        continue;
      }
      break;
    }
  }
  bool at_end() {
    ws();
    return p >= end;
  }
  bool peek(const char *s) {
    ws();
    size_t n = strlen(s);
    return (size_t)(end - p) >= n && strncmp(p, s, n) == 0;
  }
  bool accept(const char *s) {
    if (!peek(s))
      return false;
    p += strlen(s);
    return true;
  }
  void expect(const char *s) {
    if (!accept(s))
      bad(std::string("expected '") + s + "' near '" + std::string(p, std::min<size_t>(40, (size_t)(end - p))) + "'");
  }
  // identifier made of letters, digits, '_', '.', '$', '-' (not leading)
  std::string word() {
    ws();
    const char *b = p;
    while (p < end && (isalnum((unsigned char)*p) || *p == '_' || *p == '.' || *p == '$'))
      p++;
    if (b == p)
      bad("identifier expected near '" + std::string(p, std::min<size_t>(40, (size_t)(end - p))) + "'");
    return std::string(b, p);
  }
  std::string ssa() { // %name
    ws();
    if (p >= end || *p != '%')
      bad("value name expected near '" + std::string(p, std::min<size_t>(40, (size_t)(end - p))) + "'");
    p++;
    return "%" + word();
  }
  double number() {
    ws();
    char *e = nullptr;
    double v = strtod(p, &e);
    if (e == p)
      bad("number expected");
    p = e;
    return v;
  }
  std::vector<int64_t> int_list() { // [a, b, ...]
    std::vector<int64_t> v;
    expect("[");
    if (accept("]"))
      return v;
    do
      v.push_back((int64_t)number());
    while (accept(","));
    expect("]");
    return v;
  }
  // skips a balanced group that starts with `open` at the cursor
  void skip_group(char open, char close) {
    ws();
    if (p >= end || *p != open)
      bad(std::string("expected '") + open + "'");
    int depth = 0;
    for (; p < end; p++) {
      if (*p == open)
        depth++;
      else if (*p == close && !(close == '>' && p[-1] == '-') && --depth == 0) { // "->" closes nothing
        p++;
        return;
      }
    }
    bad("unbalanced brackets");
  }
  std::string group_text(char open, char close) {
    ws();
    const char *b = p;
    skip_group(open, close);
    return std::string(b + 1, p - 1);
  }
  Type type() {
    Type t;
    ws();
    if (peek("tensor<")) {
      p += 7;
      const char *b = p;
      while (p < end && *p != '>')
        p++;
      if (p >= end)
        bad("unterminated tensor type");
      std::string body(b, p);
      p++;
      t.tensor = true;
      size_t pos = 0;
      for (;;) {
        size_t x = body.find('x', pos);
        std::string part = body.substr(pos, x == std::string::npos ? std::string::npos : x - pos);
        bool num = !part.empty() && std::all_of(part.begin(), part.end(), [](char c) { return isdigit((unsigned char)c); });
        if (num && x != std::string::npos) {
          t.shape.push_back(std::stoll(part));
          pos = x + 1;
          continue;
        }
        if (part == "?" || part == "*")
          unimpl("dynamic shapes");
        t.dt = elem_type(body.substr(pos));
        break;
      }
      return t;
    }
    t.dt = elem_type(word());
    return t;
  }
};

struct Value {
  enum Kind { Tensor, Scalar, Empty } kind = Tensor;
  size_t id = 0;   // Tensor
  double scalar = 0; // Scalar
  Type type;
};

struct Builder {
  Graph g;
  std::map<std::string, Value> values;
  size_t next_id = 1u << 20; // internal tensors; arguments and results get small ids
  size_t n_args = 0;
  std::map<std::string, std::string> map_alias; // "#map1" -> "affine_map<...>"

  size_t new_tensor(const Type &t) {
    LTensor lt;
    lt.id = next_id++;
    lt.dt = t.dt;
    lt.shape = t.shape;
    g.tensors[lt.id] = lt;
    return lt.id;
  }
  const Value &val(const std::string &name) {
    auto it = values.find(name);
    if (it == values.end())
      bad("use of undefined value " + name);
    return it->second;
  }
  // the tensor behind a value that is read as an operand
  size_t operand(const std::string &name) {
    const Value &v = val(name);
    if (v.kind != Value::Tensor)
      unimpl("value " + name + " is not a computed tensor (tensor.empty or a scalar used as data)");
    return v.id;
  }
  bool is_zero_init(const std::string &name) {
    const Value &v = val(name);
    if (v.kind == Value::Empty)
      return true;
    if (v.kind == Value::Tensor) {
      const LTensor &t = g.tensors.at(v.id);
      return t.has_splat && t.splat == 0.0;
    }
    return false;
  }
  void def(const std::string &name, size_t id, const Type &t) {
    Value v;
    v.kind = Value::Tensor, v.id = id, v.type = t;
    values[name] = v;
  }
  Op &add_op(const std::string &kind, std::vector<size_t> in, size_t out) {
    Op op;
    op.kind = kind;
    op.in = std::move(in);
    op.out = {out};
    g.ops.push_back(std::move(op));
    return g.ops.back();
  }
};

Attr attr_bool(bool b) {
  Attr a;
  a.type = Attr::Bool, a.b = b;
  return a;
}
Attr attr_ints(const std::vector<int64_t> &v) {
  Attr a;
  a.type = Attr::S64Arr, a.ia = v;
  return a;
}
Attr attr_int(int64_t v) {
  Attr a;
  a.type = Attr::S64, a.i = v;
  return a;
}
Attr attr_f32(float v) {
  Attr a;
  a.type = Attr::F32, a.f = v;
  return a;
}

// affine_map<(d0, d1, d2) -> (d0, d2)>: the number of dims and, per result, the index of the dim it names.
// Results that are not a bare dim (sums, constants, symbols) are outside the subset.
struct AffineMap {
  int n_dims = 0;
  std::vector<int> res;
};

AffineMap parse_affine_map(const std::string &text) {
  Cursor c(text.c_str());
  c.expect("affine_map");
  c.expect("<");
  c.expect("(");
  AffineMap m;
  if (!c.accept(")")) {
    do {
      c.word();
      m.n_dims++;
    } while (c.accept(","));
    c.expect(")");
  }
  if (c.peek("["))
    unimpl("affine maps with symbols");
  c.expect("->");
  c.expect("(");
  if (!c.accept(")")) {
    do {
      std::string w = c.word();
      if (w.size() < 2 || w[0] != 'd' || !std::all_of(w.begin() + 1, w.end(), [](char ch) { return isdigit((unsigned char)ch); }))
        unimpl("affine map result '" + w + "' (only plain dims)");
      int d = std::stoi(w.substr(1));
      if (d >= m.n_dims)
        bad("affine map names a dim it does not declare");
      if (!c.peek(",") && !c.peek(")"))
        unimpl("affine map results that are expressions");
      m.res.push_back(d);
    } while (c.accept(","));
    c.expect(")");
  }
  c.expect(">");
  return m;
}

// the items of `key = [a, b, c]` inside an attribute dictionary, split at top-level commas
std::vector<std::string> dict_list(const std::string &dict, const std::string &key) {
  size_t k = dict.find(key);
  if (k == std::string::npos)
    bad("linalg.generic without " + key);
  size_t lb = dict.find('[', k);
  if (lb == std::string::npos)
    bad(key + " is not a list");
  std::vector<std::string> items;
  std::string cur;
  int depth = 0;
  for (size_t i = lb + 1; i < dict.size(); i++) {
    char ch = dict[i];
    if (ch == ']' && depth == 0) {
      if (!cur.empty())
        items.push_back(cur);
      return items;
    }
    if (ch == '(' || ch == '<' || ch == '[') {
      depth++;
    } else if (ch == ')' || ch == ']') {
      depth--;
    } else if (ch == '>' && !(i > 0 && dict[i - 1] == '-')) { // "->" is not a bracket
      depth--;
    }
    if (ch == ',' && depth == 0) {
      items.push_back(cur);
      cur.clear();
    } else if (!isspace((unsigned char)ch) || depth > 0) {
      cur += ch;
    }
  }
  bad(key + " is not closed");
}

// the operation names used in a region, in order, without arith.constant / linalg.yield
std::vector<std::string> region_ops(const std::string &region) {
  std::vector<std::string> ops;
  for (size_t i = 0; i + 1 < region.size(); i++) {
    if (region[i] != '=' )
      continue;
    size_t j = i + 1;
    while (j < region.size() && isspace((unsigned char)region[j]))
      j++;
    size_t e = j;
    while (e < region.size() && (isalnum((unsigned char)region[e]) || region[e] == '.' || region[e] == '_'))
      e++;
    if (e > j && region.compare(j, e - j, "arith.constant") != 0)
      ops.push_back(region.substr(j, e - j));
  }
  return ops;
}

// ins(%a, %b : T, T) / outs(%c : T): names and types
void operand_list(Cursor &c, const char *kw, std::vector<std::string> &names, std::vector<Type> &types) {
  c.expect(kw);
  c.expect("(");
  do
    names.push_back(c.ssa());
  while (c.accept(","));
  c.expect(":");
  do
    types.push_back(c.type());
  while (c.accept(","));
  c.expect(")");
  if (names.size() != types.size())
    bad(std::string(kw) + ": operand and type counts differ");
}

void parse_op(Cursor &c, Builder &b, const std::string &res, const std::string &name) {
  auto need_res = [&]() {
    if (res.empty())
      bad(name + " without a result name");
  };
  if (name == "tensor.empty") {
    need_res();
    c.expect("(");
    c.expect(")");
    c.expect(":");
    Value v;
    v.kind = Value::Empty, v.type = c.type();
    b.values[res] = v;
    return;
  }
  if (name == "arith.constant") {
    need_res();
    if (c.peek("dense<")) {
      c.p += 6;
      double x = c.number();
      c.expect(">");
      c.expect(":");
      Type t = c.type();
      size_t id = b.new_tensor(t);
      b.g.tensors[id].has_splat = true, b.g.tensors[id].splat = x;
      b.def(res, id, t);
      return;
    }
    Value v;
    v.kind = Value::Scalar;
    if (c.accept("true"))
      v.scalar = 1;
    else if (c.accept("false"))
      v.scalar = 0;
    else
      v.scalar = c.number();
    c.expect(":");
    v.type = c.type();
    b.values[res] = v;
    return;
  }
  if (name == "tensor.collapse_shape" || name == "tensor.expand_shape") {
    need_res();
    std::string src = c.ssa();
    c.skip_group('[', ']');
    if (c.accept("output_shape"))
      c.skip_group('[', ']');
    c.expect(":");
    Type from = c.type();
    c.expect("into");
    Type to = c.type();
    size_t in = b.operand(src), out = b.new_tensor(to);
    b.g.tensors[out].alias_of = (long)in;
    b.add_op("Reshape", {in}, out);
    b.def(res, out, to);
    (void)from;
    return;
  }
  if (name.rfind("onednn_graph.", 0) == 0) {
    // the reference's front-end dialect (test/mlir/test/gc/Dialect/OneDNNGraph/*.mlir): the ops of the JSON schema
    // in MLIR's generic form   %r = onednn_graph.op %a, %b {attrs} : (types) -> type
    need_res();
    static const std::map<std::string, std::string> kinds = {
        {"add", "Add"},         {"mul", "Multiply"},    {"sub", "Subtract"},        {"div", "Divide"},
        {"matmul", "MatMul"},   {"relu", "ReLU"},       {"sigmoid", "Sigmoid"},     {"pow", "Pow"},
        {"type_cast", "TypeCast"}, {"reduce_sum", "ReduceSum"}, {"reduce_mean", "ReduceMean"}};
    const std::string op = name.substr(13);
    if (!kinds.count(op))
      unimpl("operation " + name);
    std::vector<size_t> in;
    do
      in.push_back(b.operand(c.ssa()));
    while (c.accept(","));
    std::string attrs;
    if (c.peek("{"))
      attrs = c.group_text('{', '}');
    c.expect(":");
    c.expect("(");
    size_t n_types = 0;
    if (!c.accept(")")) {
      do {
        c.type();
        n_types++;
      } while (c.accept(","));
      c.expect(")");
    }
    c.expect("->");
    Type rt = c.type();
    if (n_types != in.size())
      bad(name + ": operand and type counts differ");
    Op &o = b.add_op(kinds.at(op), in, 0);
    auto flag = [&](const char *key) {
      size_t k = attrs.find(key);
      if (k == std::string::npos)
        return false;
      size_t e = attrs.find('=', k);
      return e != std::string::npos && attrs.compare(attrs.find_first_not_of(" \t\n", e + 1), 4, "true") == 0;
    };
    if (op == "matmul") {
      if (flag("transpose_a"))
        o.attrs["transpose_a"] = attr_bool(true);
      if (flag("transpose_b"))
        o.attrs["transpose_b"] = attr_bool(true);
    } else if (op == "pow") {
      size_t k = attrs.find("beta");
      if (k == std::string::npos)
        bad("onednn_graph.pow without beta");
      Cursor a(attrs.c_str() + attrs.find('=', k) + 1);
      o.attrs["beta"] = attr_f32((float)a.number());
    } else if (op == "reduce_sum" || op == "reduce_mean") {
      std::vector<int64_t> axes;
      size_t k = attrs.find("axes");
      if (k != std::string::npos) {
        size_t colon = attrs.find(':', attrs.find("array<", k));
        if (colon == std::string::npos)
          bad(name + ": axes must be array<i64: ...>");
        Cursor a(attrs.c_str() + colon + 1);
        do
          axes.push_back((int64_t)a.number());
        while (a.accept(","));
      }
      o.attrs["axes"] = attr_ints(axes);
      o.attrs["keep_dims"] = attr_bool(flag("keep_dims"));
    }
    size_t id = b.new_tensor(rt);
    b.def(res, id, rt);
    b.g.ops.back().out = {id};
    return;
  }
  if (name.rfind("linalg.", 0) != 0)
    unimpl("operation " + name);
  need_res();
  const std::string op = name.substr(7);
  // an attribute dictionary ({cast = ...}) or the short reduce form ({ arith.addf }) may follow the name
  std::string brace;
  if (c.peek("{"))
    brace = c.group_text('{', '}');
  int64_t softmax_dim = -1;
  if (op == "softmax") {
    c.expect("dimension");
    c.expect("(");
    softmax_dim = (int64_t)c.number();
    c.expect(")");
  }
  std::vector<std::string> in_names, out_names;
  std::vector<Type> in_types, out_types;
  operand_list(c, "ins", in_names, in_types);
  operand_list(c, "outs", out_names, out_types);
  std::vector<int64_t> dims;
  bool has_dims = false;
  if (c.accept("dimensions") || c.accept("permutation")) {
    c.expect("=");
    dims = c.int_list();
    has_dims = true;
  }
  std::string region;
  if (op == "generic") {
    if (c.accept("attrs")) { // attrs = {...}
      c.expect("=");
      c.skip_group('{', '}');
    }
    region = c.group_text('{', '}');
  } else if (op == "reduce" && brace.empty()) {
    c.skip_group('(', ')'); // block arguments
    region = c.group_text('{', '}');
  } else if (op == "reduce") {
    region = brace;
  }
  Type rt = out_types.at(0);
  if (c.accept("->"))
    rt = c.type();
  if (out_names.size() != 1)
    unimpl("linalg." + op + " with several results");

  auto result = [&](const Type &t) {
    size_t id = b.new_tensor(t);
    b.def(res, id, t);
    return id;
  };
  if (op == "generic") {
    // Two shapes of linalg.generic are taken: a contraction (multiply-accumulate over one reduction dim, i.e. a
    // matmul with optional batch dims and either operand transposed) and a point-wise op with identity maps.
    std::vector<AffineMap> maps;
    for (auto &item : dict_list(brace, "indexing_maps")) {
      if (!item.empty() && item[0] == '#') {
        auto it = b.map_alias.find(item);
        if (it == b.map_alias.end())
          bad("undefined affine map " + item);
        maps.push_back(parse_affine_map(it->second));
      } else {
        maps.push_back(parse_affine_map(item));
      }
    }
    std::vector<std::string> iters = dict_list(brace, "iterator_types");
    if (maps.size() != in_names.size() + 1)
      bad("linalg.generic: one indexing map per operand is needed");
    const int nd = (int)iters.size();
    for (auto &m : maps)
      if (m.n_dims != nd)
        bad("linalg.generic: map and iterator_types disagree on the number of dims");
    std::vector<int> red;
    for (int d = 0; d < nd; d++)
      if (iters[(size_t)d].find("reduction") != std::string::npos)
        red.push_back(d);
    std::vector<std::string> body = region_ops(region);
    auto identity = [&](const AffineMap &m) {
      if ((int)m.res.size() != nd)
        return false;
      for (int d = 0; d < nd; d++)
        if (m.res[(size_t)d] != d)
          return false;
      return true;
    };
    if (red.empty()) {
      static const std::map<std::string, std::string> point = {
          {"arith.addf", "Add"},      {"arith.subf", "Subtract"}, {"arith.mulf", "Multiply"}, {"arith.divf", "Divide"},
          {"arith.maximumf", "Maximum"}, {"arith.maxnumf", "Maximum"}, {"arith.negf", "Neg"},  {"math.exp", "Exp"},
          {"arith.extf", "TypeCast"}, {"arith.truncf", "TypeCast"}, {"arith.minimumf", "Minimum"}, {"arith.minnumf", "Minimum"},
          {"math.absf", "Abs"},       {"math.ceil", "Ceil"},     {"math.floor", "Floor"},    {"math.erf", "Erf"},
          {"math.log", "Log"},        {"math.round", "Round"},   {"math.rsqrt", "Rsqrt"},    {"math.sqrt", "Sqrt"},
          {"math.tanh", "Tanh"}};
      for (auto &m : maps)
        if (!identity(m))
          unimpl("point-wise linalg.generic with maps that are not the identity");
      if (body.size() != 1 || !point.count(body[0]))
        unimpl("linalg.generic body (a single arith/math op: addf, subf, mulf, divf, maximumf, minimumf, negf, extf, truncf, "
               "exp, absf, ceil, floor, erf, log, round, rsqrt, sqrt, tanh)");
      const std::string kind = point.at(body[0]);
      static const std::set<std::string> two = {"Add", "Subtract", "Multiply", "Divide", "Maximum", "Minimum"};
      const bool unary = !two.count(kind);
      if (in_names.size() != (unary ? 1u : 2u))
        bad("linalg.generic: operand count does not fit its body");
      std::vector<size_t> in;
      for (auto &n : in_names)
        in.push_back(b.operand(n));
      b.add_op(kind, in, 0);
      b.g.ops.back().out = {result(rt)};
      return;
    }
    if (red.size() != 1 || in_names.size() != 2)
      unimpl("linalg.generic with this reduction structure");
    if (!(body.size() == 2 && (body[0] == "arith.mulf" || body[0] == "arith.muli") &&
          (body[1] == "arith.addf" || body[1] == "arith.addi")))
      unimpl("linalg.generic reduction body other than multiply-accumulate");
    if (!b.is_zero_init(out_names[0]))
      unimpl("linalg.generic accumulating into a non-zero tensor");
    const int k = red[0];
    const AffineMap &ma = maps[0], &mb = maps[1], &mo = maps[2];
    const size_t ro = mo.res.size();
    if (ro < 2 || ma.res.size() != ro || mb.res.size() != ro)
      unimpl("linalg.generic contraction with broadcast operands");
    const int m = mo.res[ro - 2], n = mo.res[ro - 1];
    for (size_t d = 0; d + 2 < ro; d++) // batch dims lead, in the same order everywhere
      if (ma.res[d] != mo.res[d] || mb.res[d] != mo.res[d])
        unimpl("linalg.generic contraction with permuted batch dims");
    bool ta, tb;
    if (ma.res[ro - 2] == m && ma.res[ro - 1] == k)
      ta = false;
    else if (ma.res[ro - 2] == k && ma.res[ro - 1] == m)
      ta = true;
    else
      unimpl("linalg.generic contraction: first operand is not (m, k) or (k, m)");
    if (mb.res[ro - 2] == k && mb.res[ro - 1] == n)
      tb = false;
    else if (mb.res[ro - 2] == n && mb.res[ro - 1] == k)
      tb = true;
    else
      unimpl("linalg.generic contraction: second operand is not (k, n) or (n, k)");
    Op &o = b.add_op("MatMul", {b.operand(in_names[0]), b.operand(in_names[1])}, 0);
    if (ta)
      o.attrs["transpose_a"] = attr_bool(true);
    if (tb)
      o.attrs["transpose_b"] = attr_bool(true);
    size_t id = result(rt);
    b.g.ops.back().out = {id};
    return;
  }
  if (op == "fill") {
    const Value &v = b.val(in_names.at(0));
    if (v.kind != Value::Scalar)
      unimpl("linalg.fill of a value that is not an arith.constant");
    size_t id = result(rt);
    b.g.tensors[id].has_splat = true, b.g.tensors[id].splat = v.scalar;
    return;
  }
  if (op == "matmul" || op == "matmul_transpose_a" || op == "matmul_transpose_b" || op == "batch_matmul" ||
      op == "batch_matmul_transpose_a" || op == "batch_matmul_transpose_b") {
    if (in_names.size() != 2)
      bad("linalg." + op + " takes two inputs");
    if (!b.is_zero_init(out_names[0]))
      unimpl("linalg." + op + " accumulating into a non-zero tensor");
    Op &o = b.add_op("MatMul", {b.operand(in_names[0]), b.operand(in_names[1])}, 0);
    if (op.find("transpose_a") != std::string::npos)
      o.attrs["transpose_a"] = attr_bool(true);
    if (op.find("transpose_b") != std::string::npos)
      o.attrs["transpose_b"] = attr_bool(true);
    // the tuning attributes the reference reads from the op ({MThreads = 4 : i32, ...},
    // lib/gc/Analysis/MatmulConfigAnalysis.cpp:368-404; test/mlir/test/gc/Transforms/deepTileContractionNamedOp.mlir:33)
    for (const char *n : {"MThreads", "NThreads", "KThreads", "MBlock", "NBlock", "KBlock", "innermostMBlock",
                          "innermostNBlock", "innermostKBlock"}) {
      const std::string key = n;
      size_t at = 0;
      while ((at = brace.find(key, at)) != std::string::npos) {
        const bool starts = at == 0 || !(isalnum((unsigned char)brace[at - 1]) || brace[at - 1] == '_');
        size_t q = at + key.size();
        while (q < brace.size() && isspace((unsigned char)brace[q]))
          q++;
        if (starts && q < brace.size() && brace[q] == '=') {
          o.attrs[key] = attr_int(strtoll(brace.c_str() + q + 1, nullptr, 10));
          break;
        }
        at += key.size();
      }
    }
    size_t id = result(rt);
    b.g.ops.back().out = {id};
    return;
  }
  static const std::map<std::string, std::string> binary = {{"add", "Add"},    {"sub", "Subtract"}, {"mul", "Multiply"},
                                                            {"div", "Divide"}, {"max", "Maximum"},  {"min", "Minimum"}};
  auto splat_of = [&](const std::string &n, double &x) {
    const Value &v = b.val(n);
    if (v.kind != Value::Tensor)
      return false;
    const LTensor &t = b.g.tensors.at(v.id);
    x = t.splat;
    return t.has_splat;
  };
  if (binary.count(op)) {
    if (in_names.size() != 2)
      bad("linalg." + op + " takes two inputs");
    double x = 0;
    if (op == "max") { // max(x, 0) is the reference's ReLU (lib/gc/Transforms/OneDNNGraphToLinalg.cpp:355-358)
      for (int k = 0; k < 2; k++)
        if (splat_of(in_names[(size_t)k], x) && x == 0.0) {
          size_t in = b.operand(in_names[(size_t)(1 - k)]);
          b.add_op("ReLU", {in}, 0);
          b.g.ops.back().out = {result(rt)};
          return;
        }
    }
    size_t i0 = b.operand(in_names[0]), i1 = b.operand(in_names[1]);
    b.add_op(binary.at(op), {i0, i1}, 0);
    b.g.ops.back().out = {result(rt)};
    return;
  }
  if (op == "powf") {
    double x = 0;
    if (in_names.size() != 2 || !splat_of(in_names[1], x))
      unimpl("linalg.powf with an exponent that is not a constant");
    Op &o = b.add_op("Pow", {b.operand(in_names[0])}, 0);
    o.attrs["beta"] = attr_f32((float)x);
    b.g.ops.back().out = {result(rt)};
    return;
  }
  // the named unary ops of benchgc's linalg driver (test/benchgc/src/benchgc/linalg/eltwise.py)
  static const std::map<std::string, std::string> unary = {
      {"negf", "Neg"},   {"exp", "Exp"},     {"copy", "TypeCast"}, {"abs", "Abs"},       {"ceil", "Ceil"},
      {"floor", "Floor"}, {"erf", "Erf"},    {"log", "Log"},       {"round", "Round"},   {"rsqrt", "Rsqrt"},
      {"sqrt", "Sqrt"},  {"square", "Square"}, {"tanh", "Tanh"},   {"reciprocal", "Reciprocal"}};
  if (unary.count(op)) {
    if (in_names.size() != 1)
      bad("linalg." + op + " takes one input");
    b.add_op(unary.at(op), {b.operand(in_names[0])}, 0);
    b.g.ops.back().out = {result(rt)};
    return;
  }
  // vector forms of the contraction (test/benchgc/src/benchgc/linalg/matmul.py): a vector operand is viewed as a
  // one-row or one-column matrix and the unit dim is dropped from the result again
  if (op == "matvec" || op == "vecmat" || op == "dot" || op == "batch_matvec" || op == "batch_vecmat" ||
      op == "batch_reduce_matmul") {
    if (in_names.size() != 2)
      bad("linalg." + op + " takes two inputs");
    if (!b.is_zero_init(out_names[0]))
      unimpl("linalg." + op + " accumulating into a non-zero tensor");
    auto view = [&](size_t src, std::vector<int64_t> shape) {
      Type t;
      t.tensor = true, t.dt = b.g.tensors.at(src).dt, t.shape = std::move(shape);
      size_t v = b.new_tensor(t);
      b.g.tensors[v].alias_of = (long)src;
      b.add_op("Reshape", {src}, v);
      return v;
    };
    size_t a = b.operand(in_names[0]), w = b.operand(in_names[1]);
    const std::vector<int64_t> as = in_types[0].shape, ws = in_types[1].shape;
    std::vector<int64_t> mm_shape; // result of the matrix product before the unit dim goes
    if (op == "matvec" || op == "vecmat" || op == "dot") {
      const size_t want_a = op == "matvec" ? 2 : 1, want_w = op == "vecmat" ? 2 : 1;
      if (as.size() != want_a || ws.size() != want_w)
        bad("linalg." + op + ": operand ranks");
      // numpy matmul rules cover these as they are: [M,K]x[K] -> [M], [K]x[K,N] -> [N], [K]x[K] -> [1]
      mm_shape = op == "dot" ? std::vector<int64_t>{1} : rt.shape;
    } else if (op == "batch_matvec") {
      if (as.size() != 3 || ws.size() != 2)
        bad("linalg.batch_matvec: operand ranks");
      w = view(w, {ws[0], ws[1], 1});
      mm_shape = {as[0], as[1], 1};
    } else if (op == "batch_vecmat") {
      if (as.size() != 2 || ws.size() != 3)
        bad("linalg.batch_vecmat: operand ranks");
      a = view(a, {as[0], 1, as[1]});
      mm_shape = {ws[0], 1, ws[2]};
    } else { // batch_reduce_matmul: sum over the batch of [M,K] x [K,N]
      if (as.size() != 3 || ws.size() != 3)
        bad("linalg.batch_reduce_matmul: operand ranks");
      mm_shape = {as[0], as[1], ws[2]};
    }
    Type mt = rt;
    mt.shape = mm_shape;
    size_t prod = b.new_tensor(mt);
    b.add_op("MatMul", {a, w}, prod);
    if (op == "batch_reduce_matmul") {
      Op &o = b.add_op("ReduceSum", {prod}, 0);
      o.attrs["axes"] = attr_ints({0});
      o.attrs["keep_dims"] = attr_bool(false);
      b.g.ops.back().out = {result(rt)};
    } else if (mm_shape != rt.shape) {
      size_t v = view(prod, rt.shape);
      b.def(res, v, rt);
    } else {
      b.def(res, prod, rt);
    }
    return;
  }
  if (op == "broadcast") {
    if (!has_dims)
      bad("linalg.broadcast without dimensions");
    Op &o = b.add_op("BroadcastTo", {b.operand(in_names.at(0))}, 0);
    o.attrs["dims"] = attr_ints(dims);
    b.g.ops.back().out = {result(rt)};
    return;
  }
  if (op == "transpose") {
    if (!has_dims)
      bad("linalg.transpose without permutation");
    Op &o = b.add_op("Transpose", {b.operand(in_names.at(0))}, 0);
    o.attrs["perm"] = attr_ints(dims);
    b.g.ops.back().out = {result(rt)};
    return;
  }
  if (op == "softmax") {
    Op &o = b.add_op("SoftMax", {b.operand(in_names.at(0))}, 0);
    o.attrs["axis"] = attr_int(softmax_dim);
    b.g.ops.back().out = {result(rt)};
    return;
  }
  if (op == "reduce") {
    if (!has_dims)
      bad("linalg.reduce without dimensions");
    if (region.find("arith.addf") == std::string::npos)
      unimpl("linalg.reduce with a combiner other than arith.addf");
    if (!b.is_zero_init(out_names[0]))
      unimpl("linalg.reduce into a non-zero init");
    Op &o = b.add_op("ReduceSum", {b.operand(in_names.at(0))}, 0);
    o.attrs["axes"] = attr_ints(dims);
    o.attrs["keep_dims"] = attr_bool(false);
    b.g.ops.back().out = {result(rt)};
    return;
  }
  unimpl("operation " + name);
}

// ---- rewrites on the op list ----------------------------------------------
std::map<size_t, std::vector<size_t>> users_of(const Graph &g) {
  std::map<size_t, std::vector<size_t>> u;
  for (size_t i = 0; i < g.ops.size(); i++)
    for (auto id : g.ops[i].in)
      u[id].push_back(i);
  return u;
}

bool is_splat(const Graph &g, size_t id, double v) {
  const LTensor &t = g.tensors.at(id);
  return t.has_splat && t.splat == v;
}

// 1 / (1 + exp(-x)) written out as negf, exp, add, div becomes one Sigmoid
void fuse_sigmoid(Graph &g, const std::set<size_t> &outputs) {
  auto users = users_of(g);
  std::map<size_t, size_t> producer;
  for (size_t i = 0; i < g.ops.size(); i++)
    producer[g.ops[i].out[0]] = i;
  auto single_use = [&](size_t id) { return users[id].size() == 1 && !outputs.count(id); };
  std::set<size_t> dead;
  for (size_t i = 0; i < g.ops.size(); i++) {
    Op &d = g.ops[i];
    if (d.kind != "Divide" || !is_splat(g, d.in[0], 1.0) || !producer.count(d.in[1]))
      continue;
    size_t ia = producer[d.in[1]];
    Op &a = g.ops[ia];
    if (a.kind != "Add" || !single_use(a.out[0]))
      continue;
    size_t e_id = is_splat(g, a.in[0], 1.0) ? a.in[1] : is_splat(g, a.in[1], 1.0) ? a.in[0] : (size_t)-1;
    if (e_id == (size_t)-1 || !producer.count(e_id))
      continue;
    size_t ie = producer[e_id];
    if (g.ops[ie].kind != "Exp" || !single_use(e_id) || !producer.count(g.ops[ie].in[0]))
      continue;
    size_t in_ = producer[g.ops[ie].in[0]];
    if (g.ops[in_].kind != "Neg" || !single_use(g.ops[in_].out[0]))
      continue;
    size_t x = g.ops[in_].in[0];
    if (g.tensors.at(x).shape != g.tensors.at(d.out[0]).shape || g.tensors.at(x).dt != g.tensors.at(d.out[0]).dt)
      continue;
    d.kind = "Sigmoid";
    d.in = {x};
    d.attrs.clear();
    dead.insert(ia), dead.insert(ie), dead.insert(in_);
  }
  std::vector<Op> keep;
  for (size_t i = 0; i < g.ops.size(); i++)
    if (!dead.count(i))
      keep.push_back(g.ops[i]);
  g.ops.swap(keep);
}

// A linalg.broadcast whose users are all element-wise binary ops needs no copy: numpy broadcasting of the
// consumer does the same.  The operand is used as it is when it maps to the trailing result dimensions,
// otherwise through a view with 1s at the added dimensions.
void fold_broadcasts(Graph &g, const std::set<size_t> &outputs, size_t &next_id) {
  static const std::set<std::string> binary = {"Add", "Subtract", "Multiply", "Divide", "Maximum", "Minimum"};
  auto users = users_of(g);
  for (size_t i = 0; i < g.ops.size(); i++) {
    Op &o = g.ops[i];
    if (o.kind != "BroadcastTo" || outputs.count(o.out[0]))
      continue;
    bool ok = !users[o.out[0]].empty();
    for (size_t u : users[o.out[0]])
      ok = ok && binary.count(g.ops[u].kind);
    if (!ok)
      continue;
    const std::vector<int64_t> added = o.attrs.at("dims").ia;
    const LTensor in = g.tensors.at(o.in[0]), out = g.tensors.at(o.out[0]);
    bool leading = true;
    for (size_t k = 0; k < added.size(); k++)
      leading = leading && std::find(added.begin(), added.end(), (int64_t)k) != added.end();
    // the operand that would stand in for the broadcast: the source itself, or a view of it with unit dims
    std::vector<int64_t> repl_shape = in.shape;
    if (!leading) {
      repl_shape = out.shape;
      for (auto d : added)
        repl_shape[(size_t)d] = 1;
    }
    // every reader must still see its result shape in its operands (an op on two broadcasts of row vectors has no
    // full-shape operand left once both are folded: that broadcast stays a copy)
    for (size_t u : users[out.id]) {
      const Op &r = g.ops[u];
      std::vector<int64_t> sa = r.in[0] == out.id ? repl_shape : g.tensors.at(r.in[0]).shape,
                           sb = r.in[1] == out.id ? repl_shape : g.tensors.at(r.in[1]).shape, so;
      ok = ok && broadcast_shape(sa, sb, so) && so == g.tensors.at(r.out[0]).shape;
    }
    if (!ok)
      continue;
    size_t repl;
    if (leading) {
      repl = o.in[0];
      o.kind = "Dead";
    } else {
      LTensor v;
      v.id = next_id++;
      v.dt = in.dt;
      v.shape = out.shape;
      for (auto d : added)
        v.shape[(size_t)d] = 1;
      v.alias_of = in.has_splat ? -1 : (long)in.id;
      v.has_splat = in.has_splat, v.splat = in.splat;
      g.tensors[v.id] = v;
      repl = v.id;
      o.kind = in.has_splat ? "Dead" : "Reshape";
      o.attrs.clear();
      o.out = {v.id};
    }
    for (size_t u : users[out.id])
      for (auto &id : g.ops[u].in)
        if (id == out.id)
          id = repl;
  }
  std::vector<Op> keep;
  for (auto &o : g.ops)
    if (o.kind != "Dead")
      keep.push_back(o);
  g.ops.swap(keep);
}

// x . transpose(w) written as linalg.transpose + linalg.matmul (what exporters emit for a Linear layer) is the
// matmul with the transpose flag: the kernels read either layout in place
void fold_transposes(Graph &g) {
  std::map<size_t, size_t> producer;
  for (size_t i = 0; i < g.ops.size(); i++)
    producer[g.ops[i].out[0]] = i;
  for (auto &mm : g.ops) {
    if (mm.kind != "MatMul")
      continue;
    for (size_t side = 0; side < 2 && side < mm.in.size(); side++) {
      auto it = producer.find(mm.in[side]);
      if (it == producer.end() || g.ops[it->second].kind != "Transpose")
        continue;
      const Op &t = g.ops[it->second];
      const std::vector<int64_t> &perm = t.attrs.at("perm").ia;
      const size_t r = perm.size();
      bool last_two = r >= 2 && perm[r - 1] == (int64_t)r - 2 && perm[r - 2] == (int64_t)r - 1;
      for (size_t d = 0; d + 2 < r; d++)
        last_two = last_two && perm[d] == (int64_t)d;
      if (!last_two)
        continue;
      const char *flag = side == 0 ? "transpose_a" : "transpose_b";
      const bool was = mm.attrs.count(flag) && mm.attrs.at(flag).b;
      mm.attrs[flag] = attr_bool(!was);
      mm.in[side] = t.in[0];
    }
  }
}

void drop_dead_ops(Graph &g, const std::set<size_t> &outputs) {
  std::set<size_t> live(outputs.begin(), outputs.end());
  std::vector<char> keep(g.ops.size(), 0);
  for (size_t i = g.ops.size(); i-- > 0;) {
    if (!live.count(g.ops[i].out[0]))
      continue;
    keep[i] = 1;
    for (auto id : g.ops[i].in)
      live.insert(id);
  }
  std::vector<Op> k;
  for (size_t i = 0; i < g.ops.size(); i++)
    if (keep[i])
      k.push_back(g.ops[i]);
  g.ops.swap(k);
}

// #dlti.dl_entry<"key", value : type> entries of the module's dlti.target_system_spec
void read_target_spec(const std::string &attrs, Graph &g) {
  if (attrs.find("dlti.target_system_spec") == std::string::npos)
    return;
  const std::string tag = "#dlti.dl_entry<";
  for (size_t pos = attrs.find(tag); pos != std::string::npos; pos = attrs.find(tag, pos + 1)) {
    Cursor c(attrs.c_str() + pos + tag.size());
    c.expect("\"");
    const char *k0 = c.p;
    while (c.p < c.end && *c.p != '"')
      c.p++;
    if (c.p >= c.end)
      bad("dlti.dl_entry: unterminated key");
    std::string key(k0, c.p);
    c.p++;
    c.expect(",");
    if (c.peek("\"") || c.peek("#")) // nested specs and string values carry no number
      continue;
    double v = c.number();
    c.expect(":");
    c.word();
    c.expect(">");
    g.target_hints.emplace_back(key, (int64_t)v);
  }
}

} // namespace

Graph parse_mlir(const char *text) {
  if (!text)
    bad("null module text");
  Cursor c(text);
  Builder b;
  bool in_module = false;
  while (c.peek("#")) { // #map = affine_map<...>
    c.p++;
    std::string name = "#" + c.word();
    c.expect("=");
    c.ws();
    const char *b0 = c.p;
    c.word();
    c.skip_group('<', '>' );
    b.map_alias[name] = std::string(b0, c.p);
  }
  if (c.accept("module")) {
    if (c.accept("attributes"))
      read_target_spec(c.group_text('{', '}'), b.g);
    c.expect("{");
    in_module = true;
  }
  c.expect("func.func");
  if (c.peek("private") || c.peek("public"))
    c.word();
  c.expect("@");
  c.word();
  c.expect("(");
  if (!c.accept(")")) {
    do {
      std::string n = c.ssa();
      c.expect(":");
      Type t = c.type();
      if (!t.tensor)
        unimpl("function argument that is not a ranked tensor");
      LTensor lt;
      lt.id = b.n_args++;
      lt.dt = t.dt, lt.shape = t.shape;
      b.g.tensors[lt.id] = lt;
      b.g.input_ids.push_back(lt.id);
      b.def(n, lt.id, t);
      if (c.peek("{")) // argument attributes
        c.skip_group('{', '}');
    } while (c.accept(","));
    c.expect(")");
  }
  if (c.accept("->")) {
    if (c.peek("("))
      c.skip_group('(', ')');
    else
      c.type();
  }
  if (c.accept("attributes"))
    c.skip_group('{', '}');
  c.expect("{");
  std::vector<std::string> returned;
  for (;;) {
    if (c.at_end())
      bad("function body is not closed");
    if (c.accept("return") || c.accept("func.return")) {
      if (c.peek("%")) {
        do
          returned.push_back(c.ssa());
        while (c.accept(","));
        c.expect(":");
        do
          c.type();
        while (c.accept(","));
      }
      c.expect("}");
      break;
    }
    std::string res;
    if (c.peek("%")) {
      res = c.ssa();
      if (c.accept(":") || c.accept(","))
        unimpl("operations with several results");
      c.expect("=");
    }
    parse_op(c, b, res, c.word());
  }
  if (in_module)
    c.expect("}");

  Graph &g = b.g;
  // results: id = number of arguments + position; a returned argument, constant or repeated value is copied
  std::set<size_t> taken;
  std::map<size_t, size_t> rename;
  for (size_t j = 0; j < returned.size(); j++) {
    size_t id = b.operand(returned[j]);
    const LTensor src = g.tensors.at(id);
    const size_t want = b.n_args + j;
    if (id < b.n_args || taken.count(id) || src.has_splat || src.alias_of >= 0) {
      LTensor lt = src;
      lt.id = want, lt.has_splat = false, lt.alias_of = -1;
      g.tensors[want] = lt;
      if (src.has_splat) {
        Op &o = b.add_op("BroadcastTo", {id}, want);
        std::vector<int64_t> all(src.shape.size());
        for (size_t d = 0; d < all.size(); d++)
          all[d] = (int64_t)d;
        o.attrs["dims"] = attr_ints(all);
        LTensor one = src;
        one.shape.clear();
        g.tensors[id] = one; // the constant itself is a scalar
      } else {
        b.add_op("TypeCast", {id}, want);
      }
    } else {
      taken.insert(id);
      rename[id] = want;
    }
    g.output_ids.push_back(want);
  }
  for (auto &kv : rename) {
    LTensor lt = g.tensors.at(kv.first);
    lt.id = kv.second;
    g.tensors.erase(kv.first);
    g.tensors[kv.second] = lt;
  }
  auto rn = [&](size_t id) {
    auto it = rename.find(id);
    return it == rename.end() ? id : it->second;
  };
  for (auto &o : g.ops) {
    for (auto &id : o.in)
      id = rn(id);
    for (auto &id : o.out)
      id = rn(id);
  }
  for (auto &kv : g.tensors)
    if (kv.second.alias_of >= 0)
      kv.second.alias_of = (long)rn((size_t)kv.second.alias_of);

  std::set<size_t> outs(g.output_ids.begin(), g.output_ids.end());
  fuse_sigmoid(g, outs);
  fold_broadcasts(g, outs, b.next_id);
  fold_transposes(g);
  drop_dead_ops(g, outs);
  if (g.output_ids.empty())
    bad("the function returns nothing");
  return g;
}

} // namespace gcapi
