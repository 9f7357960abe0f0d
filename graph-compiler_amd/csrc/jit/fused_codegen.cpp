// HIP source for one fused point-wise group (see fused_jit.h).  The code follows, statement by statement, what
// fused_pointwise_kernel / fused_rowsum_kernel (kernels/eltwise.hip) do for the same parameter block.
#include <cstdlib>
#include <cstdio>
#include <cstring>
#include <sstream>

#include "fused_jit.h"

namespace gcjit {
namespace {

using gcmi::ELT_MAX_RANK;
using gcmi::FusedParams;

struct Gen {
  const FusedParams &p;
  std::ostringstream o;
  std::string idx; // type of element indices and offsets
  int W = 4;       // elements a statement block carries: 4 (quad) or 1
  explicit Gen(const FusedParams &pp) : p(pp) {}

  static std::string num(int64_t v) { return std::to_string(v) + (v > 0x7fffffffLL || v < -0x7fffffffLL ? "ll" : ""); }
  static std::string fimm(float f) { // exact: the bits
    uint32_t u;
    memcpy(&u, &f, 4);
    char b[48];
    snprintf(b, sizeof b, "__uint_as_float(0x%08xu)", u);
    return b;
  }
  static const char *ctype(int dt) { return dt == gcmi::DT_F32 ? "float" : "unsigned short"; }
  std::string reg(int v, const std::string &u) const { return "r" + std::to_string(v) + "[" + u + "]"; }

  // `var` = sum over iteration dims d_lo .. d_hi-1 of coord_d * stride[d], coords taken from `e` (innermost first)
  void offsets(const std::string &e, int d_lo, int d_hi, const std::vector<std::pair<std::string, const int64_t *>> &targets,
               const std::string &ind) {
    if (targets.empty())
      return;
    if (d_hi - d_lo == 1) {
      for (auto &t : targets)
        if (t.second[d_lo] != 0)
          o << ind << t.first << " += (" << idx << ")(" << e << ") * (" << idx << ")" << num(t.second[d_lo]) << ";\n";
      return;
    }
    o << ind << "{ " << idx << " rem_ = " << e << ", c_;\n";
    for (int d = d_hi - 1; d >= d_lo; d--) {
      if (d > d_lo)
        o << ind << "  c_ = rem_ % (" << idx << ")" << num(p.dims[d]) << "; rem_ /= (" << idx << ")" << num(p.dims[d]) << ";\n";
      else
        o << ind << "  c_ = rem_;\n";
      for (auto &t : targets)
        if (t.second[d] != 0)
          o << ind << "  " << t.first << " += c_ * (" << idx << ")" << num(t.second[d]) << ";\n";
    }
    o << ind << "}\n";
  }

  // inputs k0 .. k1-1 at offsets off<k> into registers r<k>[0..W); `held` inputs are not loaded (see keep_from)
  std::vector<int> keep_from; // second-pass input k -> the first-pass input whose values are still in registers, or -1
  void loads(int k0, int k1, const std::string &ind, bool skip_held = false) {
    const int last = ELT_MAX_RANK - 1;
    for (int k = k0; k < k1; k++) {
      if (skip_held && keep_from[(size_t)k] >= 0)
        continue;
      const bool f32 = p.in_dt[k] == gcmi::DT_F32, vec = W == 4 && ((p.vec_mask >> k) & 1);
      const std::string src = "reinterpret_cast<const " + std::string(ctype(p.in_dt[k])) + " *>(in" + std::to_string(k) + ")";
      o << ind << "float r" << k << "[" << W << "];\n";
      auto conv = [&](const std::string &raw) {
        if (f32)
          return raw;
        if (p.in_dt[k] == gcmi::DT_BF16)
          return "gcmi::bf16_bits_to_f32(" + raw + ")";
        return "(float)__builtin_bit_cast(_Float16, (unsigned short)(" + raw + "))";
      };
      if (vec && f32) {
        o << ind << "{ const f4_ q_ = *reinterpret_cast<const f4_ *>(" << src << " + off" << k << ");"
          << " r" << k << "[0] = q_[0]; r" << k << "[1] = q_[1]; r" << k << "[2] = q_[2]; r" << k << "[3] = q_[3]; }\n";
      } else if (vec) {
        o << ind << "{ const u2_ q_ = *reinterpret_cast<const u2_ *>(" << src << " + off" << k << ");\n";
        o << ind << "  r" << k << "[0] = " << conv("(unsigned short)q_[0]") << "; r" << k << "[1] = " << conv("(unsigned short)(q_[0] >> 16)")
          << "; r" << k << "[2] = " << conv("(unsigned short)q_[1]") << "; r" << k << "[3] = " << conv("(unsigned short)(q_[1] >> 16)") << "; }\n";
      } else if (W == 4) {
        const int64_t step = p.in_str[k][last];
        if (step == 0) { // a broadcast along the innermost dim: one load
          o << ind << "{ const float s_ = " << conv(src + "[off" + std::to_string(k) + "]") << ";"
            << " r" << k << "[0] = s_; r" << k << "[1] = s_; r" << k << "[2] = s_; r" << k << "[3] = s_; }\n";
        } else {
          for (int u = 0; u < 4; u++)
            o << ind << "r" << k << "[" << u << "] = "
              << conv(src + "[(long long)off" + std::to_string(k) + " + " + num((int64_t)u * step) + "]") << ";\n";
        }
      } else {
        o << ind << "r" << k << "[0] = " << conv(src + "[off" + std::to_string(k) + "]") << ";\n";
      }
      if (!f32) // the widened value is opaque to the ops that read it (see ops())
        for (int u = 0; u < W; u++)
          o << ind << "asm volatile(\"\" : \"+v\"(r" << k << "[" << u << "]));\n";
    }
  }

  // instructions j0 .. j1-1 on registers of width w (1 for per-row values)
  void ops(int j0, int j1, int w, const std::string &ind) {
    for (int j = j0; j < j1; j++) {
      const gcmi::FusedIns &in = p.ins[j];
      const int v = p.n_in + j;
      o << ind << "float r" << v << "[" << w << "];\n";
      for (int u = 0; u < w; u++) {
        // a per-row register (width 1) read by a per-element instruction: the same value for every element
        auto src = [&](int r) {
          const bool row_value = width_of(r) == 1;
          return "r" + std::to_string(r) + "[" + (row_value ? "0" : std::to_string(u)) + "]";
        };
        const std::string x = src(in.a), y = src(in.b), d = "r" + std::to_string(v) + "[" + std::to_string(u) + "]";
        std::string e;
        switch (in.op) {
        case gcmi::ELT_ADD: e = x + " + " + y; break;
        case gcmi::ELT_SUB: e = x + " - " + y; break;
        case gcmi::ELT_MUL: e = x + " * " + y; break;
        case gcmi::ELT_DIV: e = x + " / " + y; break;
        case gcmi::ELT_NEG: e = "-" + x; break;
        case gcmi::ELT_SQUARE: e = x + " * " + x; break;
        case gcmi::ELT_COPY: e = x; break;
        default: e = "gcmi::fused_op(" + std::to_string(in.op) + ", " + x + ", " + y + ", " + fimm(in.imm) + ")"; break;
        }
        // Every op stands alone, as in the library kernel where its operands come out of LDS: a barrier keeps the
        // compiler from contracting a multiply into the next op's add, or from narrowing f16 -> sqrt -> f16 to a
        // half-precision instruction with other rounding.
        o << ind << d << " = " << e << ";\n";
        if (in.dt == gcmi::DT_BF16 || in.dt == gcmi::DT_F16)
          o << ind << "asm volatile(\"\" : \"+v\"(" << d << "));\n";
        if (in.dt == gcmi::DT_BF16)
          o << ind << d << " = gcmi::bf16_bits_to_f32(gcmi::f32_to_bf16_bits(" << d << "));\n";
        else if (in.dt == gcmi::DT_F16)
          o << ind << d << " = (float)(_Float16)" << d << ";\n";
        o << ind << "asm volatile(\"\" : \"+v\"(" << d << "));\n";
      }
    }
  }

  // width of the C array that holds register r (set while a kernel is written)
  std::vector<int> widths;
  int width_of(int r) const { return widths[(size_t)r]; }

  void store(const std::string &ptr, int dt, bool vec, int64_t step, const std::string &off, int reg_v, const std::string &ind) {
    const std::string dst = "reinterpret_cast<" + std::string(ctype(dt)) + " *>(" + ptr + ")";
    auto val = [&](int u) { return "r" + std::to_string(reg_v) + "[" + (width_of(reg_v) == 1 ? "0" : std::to_string(u)) + "]"; };
    auto conv = [&](const std::string &v) {
      if (dt == gcmi::DT_F32)
        return v;
      if (dt == gcmi::DT_BF16)
        return "gcmi::f32_to_bf16_bits(" + v + ")";
      return "__builtin_bit_cast(unsigned short, (_Float16)" + v + ")";
    };
    if (W == 1) {
      o << ind << dst << "[" << off << "] = " << conv(val(0)) << ";\n";
    } else if (vec && dt == gcmi::DT_F32) {
      o << ind << "*reinterpret_cast<f4_ *>(" << dst << " + " << off << ") = f4_{" << val(0) << ", " << val(1) << ", " << val(2) << ", "
        << val(3) << "};\n";
    } else if (vec) {
      o << ind << "*reinterpret_cast<u2_ *>(" << dst << " + " << off << ") = u2_{(unsigned)" << conv(val(0)) << " | ((unsigned)"
        << conv(val(1)) << " << 16), (unsigned)" << conv(val(2)) << " | ((unsigned)" << conv(val(3)) << " << 16)};\n";
    } else {
      for (int u = 0; u < 4; u++)
        o << ind << dst << "[(long long)" << off << " + " << num((int64_t)u * step) << "] = " << conv(val(u)) << ";\n";
    }
  }

  void signature(const std::string &name, int threads) {
    o << "extern \"C\" __global__ __launch_bounds__(" << threads << ") void " << name << "(";
    for (int k = 0; k < p.n_in; k++)
      o << "const void *__restrict__ in" << k << ", ";
    o << "void *__restrict__ out) {\n";
  }
};

bool wide_indices(const FusedParams &p) {
  if (p.n >= ((int64_t)1 << 31))
    return true;
  for (int k = 0; k <= p.n_in; k++) {
    int64_t far = 0;
    for (int d = 0; d < ELT_MAX_RANK; d++) {
      const int64_t st = k < p.n_in ? p.in_str[k][d] : p.out_str[d];
      if (st < 0)
        return true;
      far += (p.dims[d] - 1) * st;
    }
    if (far + 4 >= ((int64_t)1 << 31))
      return true;
  }
  return false;
}

} // namespace

bool generate_fused(const FusedParams &raw, const int *same_as, const std::string &name, FusedKernelSource &out) {
  FusedParams p = raw;
  if (p.n <= 0 || gcmi::fused_prepare(p, true) != 0)
    return false;
  const bool has_sum = p.sum_ins >= 0, second_pass = has_sum && p.row_end < p.n_ins;
  Gen g(p);
  g.idx = wide_indices(p) ? "long long" : "unsigned";
  g.W = p.quad ? 4 : 1;
  g.widths.assign((size_t)(p.n_in + p.n_ins), g.W);
  const int d0 = ELT_MAX_RANK - p.rank, last = ELT_MAX_RANK - 1;
  std::ostringstream &o = g.o;
  out.name = name, out.n_in = p.n_in, out.quad = p.quad != 0;

  if (!has_sum) {
    const int threads = 256;
    const int64_t chunk = 4 * threads, steps = (p.n + chunk - 1) / chunk;
    const int64_t blocks = steps < ((int64_t)1 << 20) ? steps : (int64_t)1 << 20;
    out.grid = (unsigned)blocks, out.block = threads;
    g.signature(name, threads);
    o << "  for (long long c0 = (long long)blockIdx.x * " << chunk << "; c0 < " << p.n << "ll; c0 += " << blocks * chunk << "ll) {\n";
    auto body = [&](const std::string &e, const std::string &ind) {
      std::vector<std::pair<std::string, const int64_t *>> t;
      std::vector<std::string> names((size_t)p.n_in);
      for (int k = 0; k < p.n_in; k++) {
        names[(size_t)k] = "off" + std::to_string(k);
        o << ind << g.idx << " off" << k << " = 0;\n";
        t.emplace_back(names[(size_t)k], p.in_str[k]);
      }
      g.offsets(e, d0, ELT_MAX_RANK, t, ind);
      g.loads(0, p.n_in, ind);
      g.ops(0, p.n_ins, g.W, ind);
      g.store("out", p.out_dt, p.out_vec != 0, 1, e, p.out_reg, ind); // the output is dense
    };
    if (p.quad) {
      o << "    const long long e_ = c0 + 4 * (long long)threadIdx.x;\n    if (e_ < " << p.n << "ll) {\n      const " << g.idx
        << " e = (" << g.idx << ")e_;\n";
      body("e", "      ");
      o << "    }\n";
    } else {
      o << "#pragma unroll\n    for (int u = 0; u < 4; u++) {\n      const long long e_ = c0 + (long long)u * " << threads
        << " + threadIdx.x;\n      if (e_ < " << p.n << "ll) {\n        const " << g.idx << " e = (" << g.idx << ")e_;\n";
      body("e", "        ");
      o << "      }\n    }\n";
    }
    o << "  }\n}\n";
    out.source = o.str();
    return true;
  }

  // ---- a row kernel: the launch shapes of gcmi_launch_fused, so that partial sums are formed in the same order
  const int64_t rows = p.n / p.n_red;
  if (rows > 0x7fffffff)
    return false;
  int threads, tpr;
  {
    FusedParams q = p;
    if (gcmi::fused_allocate(q) > gcmi::FUSED_MAX_PHYS)
      return false;
    const size_t per_thread = (size_t)q.n_phys * sizeof(float) * 4, room = 65536 - sizeof(FusedParams) - 512;
    if (rows < 512 && p.n_red >= 2048 && per_thread * 512 <= room)
      threads = 512, tpr = 512;
    else if (p.n_red >= 512 || rows < 64)
      threads = 256, tpr = 256;
    else
      threads = 256, tpr = 64;
  }
  const int rows_per_wg = threads / tpr;
  out.grid = (unsigned)((rows + rows_per_wg - 1) / rows_per_wg), out.block = (unsigned)threads;
  const int d_row = ELT_MAX_RANK - p.rank_red;
  const int sum_v = p.n_in + p.sum_ins, sum_a = p.ins[p.sum_ins].a, sum_dt = p.ins[p.sum_ins].dt;
  // widths: per-row values (the sum, the per-row inputs, the instructions of the row phase) are single floats
  g.widths[(size_t)sum_v] = 1;
  for (int k = p.n_in_pre; k < p.n_in_row; k++)
    g.widths[(size_t)k] = 1;
  for (int j = p.sum_ins + 1; j < p.row_end; j++)
    g.widths[(size_t)(p.n_in + j)] = 1;

  g.signature(name, threads);
  if (tpr > 64)
    o << "  __shared__ float wave_sum[" << threads / 64 << "];\n";
  o << "  const int tid = threadIdx.x, sub = tid % " << tpr << ";\n";
  o << "  const long long row_raw = (long long)blockIdx.x * " << rows_per_wg << " + tid / " << tpr << ";\n";
  o << "  const bool live = row_raw < " << rows << "ll;\n";
  o << "  const " << g.idx << " row = (" << g.idx << ")(live ? row_raw : " << rows - 1 << "ll);\n";
  {
    std::vector<std::pair<std::string, const int64_t *>> t;
    std::vector<std::string> names;
    for (int k = 0; k < p.n_in; k++) {
      o << "  " << g.idx << " base" << k << " = 0;\n";
      names.push_back("base" + std::to_string(k));
    }
    for (int k = 0; k < p.n_in; k++)
      t.emplace_back(names[(size_t)k], p.in_str[k]);
    if (second_pass) {
      o << "  " << g.idx << " obase = 0;\n";
      t.emplace_back("obase", p.out_str);
    }
    g.offsets("row", d0, d_row, t, "  ");
  }
  const int64_t step_elems = (int64_t)tpr * 4, trips = (p.n_red + step_elems - 1) / step_elems;
  // A second-pass input that is a first-pass input again (the row that is normalised) is not read twice when a
  // thread's share of the row is small enough to stay in registers.
  g.keep_from.assign((size_t)p.n_in, -1);
  std::vector<char> kept((size_t)p.n_in, 0);
  if (second_pass && same_as && trips <= 8)
    for (int k = p.n_in_row; k < p.n_in; k++)
      if (same_as[k] >= 0 && same_as[k] < p.n_in_pre)
        g.keep_from[(size_t)k] = same_as[k], kept[(size_t)same_as[k]] = 1;
  for (int k = 0; k < p.n_in_pre; k++)
    if (kept[(size_t)k])
      o << "  float keep" << k << "[" << trips << "][" << g.W * (p.quad ? 1 : 4) << "] = {};\n";
  auto row_loop = [&](int k0, int k1, int j0, int j1, bool pass2) {
    if (trips <= 8)
      o << "#pragma unroll\n";
    o << "  for (int it_ = 0; it_ < " << trips << "; it_++) {\n    const " << g.idx << " s0_ = (" << g.idx << ")it_ * " << step_elems
      << ";\n";
    auto body = [&](const std::string &e, const std::string &ind) {
      std::vector<std::pair<std::string, const int64_t *>> t;
      std::vector<std::string> names;
      for (int k = k0; k < k1; k++) {
        o << ind << g.idx << " off" << k << " = base" << k << ";\n";
        names.push_back("off" + std::to_string(k));
      }
      for (int k = k0; k < k1; k++)
        t.emplace_back(names[(size_t)(k - k0)], p.in_str[k]);
      if (pass2) {
        o << ind << g.idx << " ooff = obase;\n";
        t.emplace_back("ooff", p.out_str);
      }
      g.offsets(e, d_row, ELT_MAX_RANK, t, ind);
      g.loads(k0, k1, ind, pass2);
      // quad: a thread's four elements of the step; otherwise element u of the step (the loop variable around this body)
      for (int k = k0; k < k1; k++) {
        const std::string slot = p.quad ? "" : "u * 1 + ";
        if (!pass2 && kept[(size_t)k])
          for (int u = 0; u < g.W; u++)
            o << ind << "keep" << k << "[it_][" << slot << u << "] = r" << k << "[" << u << "];\n";
        if (pass2 && g.keep_from[(size_t)k] >= 0) {
          o << ind << "float r" << k << "[" << g.W << "];\n";
          for (int u = 0; u < g.W; u++)
            o << ind << "r" << k << "[" << u << "] = keep" << g.keep_from[(size_t)k] << "[it_][" << slot << u << "];\n";
        }
      }
      g.ops(j0, j1, g.W, ind);
      if (!pass2) {
        for (int u = 0; u < g.W; u++)
          o << ind << "acc += r" << sum_a << "[" << u << "];\n";
      } else {
        o << ind << "if (live) {\n";
        g.store("out", p.out_dt, p.out_vec != 0, p.out_str[last], "ooff", p.out_reg, ind + "  ");
        o << ind << "}\n";
      }
    };
    if (p.quad) {
      o << "    const " << g.idx << " e = s0_ + 4 * (" << g.idx << ")sub;\n    if (e < (" << g.idx << ")" << Gen::num(p.n_red) << ") {\n";
      body("e", "      ");
      o << "    }\n";
    } else {
      o << "#pragma unroll\n    for (int u = 0; u < 4; u++) {\n      const " << g.idx << " e = s0_ + (" << g.idx << ")u * " << tpr
        << " + (" << g.idx << ")sub;\n      if (e < (" << g.idx << ")" << Gen::num(p.n_red) << ") {\n";
      body("e", "        ");
      o << "      }\n    }\n";
    }
    o << "  }\n";
  };
  o << "  float acc = 0.0f;\n";
  row_loop(0, p.n_in_pre, 0, p.sum_ins, false);
  o << "#pragma unroll\n  for (int s = 32; s > 0; s >>= 1)\n    acc += __shfl_xor(acc, s);\n";
  if (tpr > 64) {
    o << "  if ((tid & 63) == 0)\n    wave_sum[tid >> 6] = acc;\n  __syncthreads();\n  acc = 0.0f;\n";
    o << "  { const int w0 = (tid / " << tpr << ") * " << tpr / 64 << ";\n";
    o << "    for (int w = 0; w < " << tpr / 64 << "; w++)\n      acc += wave_sum[w0 + w]; }\n";
  }
  if (p.mean)
    o << "  acc = acc / (float)" << p.n_red << "ll;\n";
  if (sum_dt == gcmi::DT_BF16)
    o << "  acc = gcmi::bf16_bits_to_f32(gcmi::f32_to_bf16_bits(acc));\n";
  else if (sum_dt == gcmi::DT_F16)
    o << "  acc = (float)(_Float16)acc;\n";
  o << "  float r" << sum_v << "[1] = {acc};\n  asm volatile(\"\" : \"+v\"(r" << sum_v << "[0]));\n";
  // per-row inputs, the instructions of the row
  {
    const int keepW = g.W;
    g.W = 1;
    for (int k = p.n_in_pre; k < p.n_in_row; k++)
      o << "  const " << g.idx << " off" << k << " = base" << k << ";\n";
    g.loads(p.n_in_pre, p.n_in_row, "  ");
    g.ops(p.sum_ins + 1, p.row_end, 1, "  ");
    if (!second_pass) {
      o << "  if (sub == 0 && live) {\n";
      g.store("out", p.out_dt, false, 1, "row", p.out_reg, "    ");
      o << "  }\n";
    }
    g.W = keepW;
  }
  if (second_pass)
    row_loop(p.n_in_row, p.n_in, p.row_end, p.n_ins, true);
  o << "}\n";
  out.source = o.str();
  return true;
}

} // namespace gcjit
