// HIP source for a softmax over the innermost axis of one shape (see fused_jit.h): the library's softmax_kernel
// (kernels/eltwise.hip) gives a wave to a row and walks it three times with one element per lane and load; here a
// row is loaded once, four elements per lane and load, by as many threads as keep a thread's share in registers,
// and written once.  max, x - max, exp, sum, divide: the decomposition of
// lib/gc/Transforms/DecomposeAggregatedOps.cpp:24-38, in f32 whatever the storage type.
#include <sstream>

#include "fused_jit.h"

namespace gcjit {

bool generate_softmax(int64_t rows, int64_t len, int in_dt, int out_dt, const std::string &name, FusedKernelSource &out) {
  auto is_float = [](int dt) { return dt == gcmi::DT_F32 || dt == gcmi::DT_BF16 || dt == gcmi::DT_F16; };
  if (rows < 1 || len < 1 || rows > 0x7fffffff || !is_float(in_dt) || !is_float(out_dt))
    return false;
  // threads per row: a thread holds at most 32 elements
  int tpr;
  if (len <= 512)
    tpr = 64;
  else if (len <= 8192)
    tpr = 256;
  else if (len <= 32768)
    tpr = 1024;
  else
    return false;
  const int threads = tpr < 256 ? 256 : tpr, rows_per_wg = threads / tpr, waves_per_row = tpr / 64;
  const bool quad = len % 4 == 0;
  const int w = quad ? 4 : 1;
  const int64_t step = (int64_t)tpr * w, trips = (len + step - 1) / step;
  const bool wide = rows * len >= ((int64_t)1 << 31);
  const char *idx = wide ? "long long" : "unsigned";
  auto ctype = [](int dt) { return dt == gcmi::DT_F32 ? "float" : "unsigned short"; };
  auto widen = [&](const std::string &raw) {
    if (in_dt == gcmi::DT_F32)
      return raw;
    if (in_dt == gcmi::DT_BF16)
      return "gcmi::bf16_bits_to_f32((unsigned short)(" + raw + "))";
    return "(float)__builtin_bit_cast(_Float16, (unsigned short)(" + raw + "))";
  };
  auto narrow = [&](const std::string &v) {
    if (out_dt == gcmi::DT_F32)
      return v;
    if (out_dt == gcmi::DT_BF16)
      return "gcmi::f32_to_bf16_bits(" + v + ")";
    return "__builtin_bit_cast(unsigned short, (_Float16)(" + v + "))";
  };
  std::ostringstream o;
  o << "extern \"C\" __global__ __launch_bounds__(" << threads << ") void " << name
    << "(const void *__restrict__ in0, void *__restrict__ out) {\n";
  if (waves_per_row > 1)
    o << "  __shared__ float part[2][" << threads / 64 << "];\n";
  o << "  const int tid = threadIdx.x, sub = tid % " << tpr << ";\n";
  o << "  const long long row_raw = (long long)blockIdx.x * " << rows_per_wg << " + tid / " << tpr << ";\n";
  o << "  const bool live = row_raw < " << rows << "ll;\n";
  o << "  const " << idx << " base = (" << idx << ")(live ? row_raw : " << rows - 1 << "ll) * (" << idx << ")" << len << ";\n";
  o << "  const " << ctype(in_dt) << " *src = reinterpret_cast<const " << ctype(in_dt) << " *>(in0) + base;\n";
  o << "  " << ctype(out_dt) << " *dst = reinterpret_cast<" << ctype(out_dt) << " *>(out) + base;\n";
  o << "  float v[" << trips << "][" << w << "];\n  float m = -__builtin_inff();\n";
  // load, row maximum
  o << "#pragma unroll\n  for (int it = 0; it < " << trips << "; it++) {\n";
  o << "    const long long e = (long long)it * " << step << " + (long long)sub * " << w << ";\n";
  o << "    if (e < " << len << "ll) {\n";
  if (quad && in_dt == gcmi::DT_F32) {
    o << "      const f4_ q = *reinterpret_cast<const f4_ *>(src + e);\n";
    for (int u = 0; u < 4; u++)
      o << "      v[it][" << u << "] = q[" << u << "];\n";
  } else if (quad) {
    o << "      const u2_ q = *reinterpret_cast<const u2_ *>(src + e);\n";
    o << "      v[it][0] = " << widen("q[0]") << "; v[it][1] = " << widen("q[0] >> 16") << "; v[it][2] = " << widen("q[1]")
      << "; v[it][3] = " << widen("q[1] >> 16") << ";\n";
  } else {
    o << "      v[it][0] = " << widen("src[e]") << ";\n";
  }
  for (int u = 0; u < w; u++)
    o << "      m = fmaxf(m, v[it][" << u << "]);\n";
  o << "    } else {\n";
  for (int u = 0; u < w; u++)
    o << "      v[it][" << u << "] = -__builtin_inff();\n";
  o << "    }\n  }\n";
  auto reduce = [&](const char *var, const char *op, int buf) {
    o << "#pragma unroll\n  for (int s = 32; s > 0; s >>= 1)\n    " << var << " = " << op << "(" << var << ", __shfl_xor(" << var
      << ", s));\n";
    if (waves_per_row > 1) {
      o << "  if ((tid & 63) == 0)\n    part[" << buf << "][tid >> 6] = " << var << ";\n  __syncthreads();\n";
      o << "  { const int w0 = (tid / " << tpr << ") * " << waves_per_row << ";\n    " << var << " = part[" << buf << "][w0];\n";
      o << "    for (int k = 1; k < " << waves_per_row << "; k++)\n      " << var << " = " << op << "(" << var << ", part[" << buf
        << "][w0 + k]); }\n";
    }
  };
  o << "  auto add_ = [](float a, float b) { return a + b; };\n";
  reduce("m", "fmaxf", 0);
  // exponentials and their sum (elements past the row are exp(-inf) = 0)
  o << "  float sum = 0.0f;\n#pragma unroll\n  for (int it = 0; it < " << trips << "; it++) {\n";
  for (int u = 0; u < w; u++)
    o << "    v[it][" << u << "] = expf(v[it][" << u << "] - m);\n    sum += v[it][" << u << "];\n";
  o << "  }\n";
  reduce("sum", "add_", 1);
  // scale and store
  o << "#pragma unroll\n  for (int it = 0; it < " << trips << "; it++) {\n";
  o << "    const long long e = (long long)it * " << step << " + (long long)sub * " << w << ";\n";
  o << "    if (live && e < " << len << "ll) {\n";
  if (quad && out_dt == gcmi::DT_F32) {
    o << "      *reinterpret_cast<f4_ *>(dst + e) = f4_{v[it][0] / sum, v[it][1] / sum, v[it][2] / sum, v[it][3] / sum};\n";
  } else if (quad) {
    o << "      *reinterpret_cast<u2_ *>(dst + e) = u2_{(unsigned)" << narrow("v[it][0] / sum") << " | ((unsigned)"
      << narrow("v[it][1] / sum") << " << 16), (unsigned)" << narrow("v[it][2] / sum") << " | ((unsigned)" << narrow("v[it][3] / sum")
      << " << 16)};\n";
  } else {
    o << "      dst[e] = " << narrow("v[it][0] / sum") << ";\n";
  }
  o << "    }\n  }\n}\n";
  out.name = name, out.source = o.str(), out.n_in = 1, out.quad = quad;
  out.grid = (unsigned)((rows + rows_per_wg - 1) / rows_per_wg), out.block = (unsigned)threads;
  return true;
}

} // namespace gcjit
