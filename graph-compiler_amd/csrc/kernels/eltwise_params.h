// Argument blocks of the generic element-wise / reduce / softmax kernels.
#pragma once
#include <stdint.h>
#include "op_codes.h"

namespace gcmi {

static constexpr int ELT_MAX_RANK = 6;

struct EltParams {
  const void *a;
  const void *b; // null for unary ops
  void *out;     // dense row-major over dims
  int64_t n;
  int64_t dims[ELT_MAX_RANK]; // left-padded with 1
  int64_t sa[ELT_MAX_RANK];   // element strides of a (0 on broadcast dims)
  int64_t sb[ELT_MAX_RANK];
  int32_t op, a_dt, b_dt, out_dt;
  float alpha;          // Pow exponent
  const float *scales;  // (de)quantise: device arrays
  const int32_t *zps;
  int32_t n_scales, ch_axis; // ch_axis indexes dims[] (after left padding)
};

struct ReduceParams {
  const void *in;
  void *out;
  int64_t n_out, n_red;
  int64_t kdims[ELT_MAX_RANK], kstr[ELT_MAX_RANK]; // kept dims and their input strides
  int64_t rdims[ELT_MAX_RANK], rstr[ELT_MAX_RANK]; // reduced dims and their input strides
  int32_t dt, mean;
};

// A group of point-wise ops fused into one launch: a straight-line program over f32 registers, evaluated once per
// element of the iteration space.  As handed to the launcher the program is in single-assignment form: registers
// 0 .. n_in-1 are the inputs (read through broadcast strides), instruction j writes register n_in + j.  Every
// instruction rounds its result to the storage type its op has in the graph (dt), so the fused group computes bit
// for bit what the ops compute one launch at a time.
//
// With a sum inside (sum_ins >= 0) the iteration space is [n / n_red rows, n_red]:
//   1. instructions before sum_ins run per element and read inputs 0 .. n_in_pre-1;
//   2. instruction sum_ins (ELT_ROWSUM) is the sum (or mean) over the row of its register a; instructions
//      sum_ins+1 .. row_end-1 run once per row and may read inputs n_in_pre .. n_in_row-1 (stride 0 along the row);
//   3. instructions row_end .. n_ins-1, if any, run per element again -- a second pass over the row that may read
//      inputs n_in_row .. n_in-1 and every per-row value of step 2 (not the per-element values of step 1) and
//      writes an output of the full shape through out_str.  Without step 3 the output has one value per row.
// A normalisation (row statistic, then scaling by it) is one launch this way.
//
// The launcher maps the registers onto as few physical ones as their lifetimes allow (fused_allocate below): the
// kernels keep them in LDS, four elements of a thread side by side, and fewer registers mean more workgroups per
// compute unit.
static constexpr int FUSED_MAX_IN = 8, FUSED_MAX_INS = 16;
static constexpr int FUSED_MAX_PHYS = 15; // 15 x 256 threads x 16 bytes + the parameter block fit 64 KiB of LDS

struct FusedIns {
  int32_t op;   // EltOp (not the (de)quantise ops)
  int32_t a, b; // source registers (b unused by unary ops)
  int32_t dt;   // storage type of the result: DT_F32 / DT_BF16 / DT_F16
  float imm;    // Pow exponent
  int32_t d;    // destination register (set by the launcher)
};

struct FusedParams {
  const void *in[FUSED_MAX_IN];
  void *out;
  int64_t in_str[FUSED_MAX_IN][ELT_MAX_RANK]; // element strides per iteration dim (0 on broadcast dims)
  int64_t dims[ELT_MAX_RANK];                 // iteration space, left-padded with 1
  int64_t n;                                  // its element count
  int64_t n_red;                              // row length (1 without a sum)
  int64_t out_str[ELT_MAX_RANK];              // second pass: element strides of the output per iteration dim
  int32_t in_dt[FUSED_MAX_IN];
  int32_t out_dt, out_reg;
  int32_t n_in, n_in_pre, n_ins, sum_ins; // sum_ins: -1 without a sum
  int32_t n_in_row, row_end;              // see above; n_in_row = n_in and row_end = n_ins without a second pass
  int32_t mean;
  // set by the launcher
  int32_t rank, rank_red;          // dims after merging, and how many of them lie inside a row
  int32_t quad, vec_mask, out_vec; // four-element groups; inputs / output that move as 16- or 8-byte vectors
  int32_t in_reg[FUSED_MAX_IN];    // physical register of each input
  int32_t n_phys;                  // physical registers in use
  FusedIns ins[FUSED_MAX_INS];
};

// Validates a fused program and brings its iteration space into the form the kernels walk: neighbouring dims merged,
// the four-element mode and the vector moves decided, the dims inside a row counted.  Returns 0, or 2 for a
// program that is not well formed.  assume_aligned: decide the vector moves from the strides alone (for code that is
// generated before the addresses are known and checks them when it is launched).
inline int fused_prepare(FusedParams &p, bool assume_aligned) {
  enum { PDT_F16 = 1, PDT_BF16 = 2, PDT_F32 = 3 }; // dnnl_data_type_t values, as everywhere in these parameter blocks
  const bool has_sum = p.sum_ins >= 0;
  if (p.n_in < 1 || p.n_in > FUSED_MAX_IN || p.n_ins < 0 || p.n_ins > FUSED_MAX_INS || p.sum_ins >= p.n_ins)
    return 2;
  if (!has_sum)
    p.n_in_pre = p.n_in_row = p.n_in, p.row_end = p.n_ins, p.n_red = 1;
  if (p.n_in_pre < 0 || p.n_in_pre > p.n_in_row || p.n_in_row > p.n_in || p.n_red < 1 || p.n % p.n_red != 0 ||
      (has_sum && (p.row_end <= p.sum_ins || p.row_end > p.n_ins)))
    return 2;
  auto is_float = [](int dt) { return dt == PDT_F32 || dt == PDT_BF16 || dt == PDT_F16; };
  for (int k = 0; k < p.n_in; k++)
    if (!is_float(p.in_dt[k]) || (!p.in[k] && !assume_aligned))
      return 2;
  if (!is_float(p.out_dt) || (!p.out && !assume_aligned))
    return 2;
  const bool second_pass = has_sum && p.row_end < p.n_ins;
  if (!second_pass && p.n_in_row != p.n_in)
    return 2;
  // every instruction reads registers that are already written and that exist in its phase: before the sum the
  // per-element inputs and results; per row the sum, the per-row inputs and results; in the second pass the
  // per-row values, its own inputs and results
  auto phase_of_ins = [&](int j) { return !has_sum ? 0 : j < p.sum_ins ? 0 : j < p.row_end ? 1 : 2; };
  auto readable = [&](int r, int j) {
    if (r < 0 || r >= p.n_in + j)
      return false;
    if (!has_sum)
      return true;
    const int ph = j <= p.sum_ins ? 0 : phase_of_ins(j); // the sum itself reads a per-element value
    const int src = r < p.n_in ? (r < p.n_in_pre ? 0 : r < p.n_in_row ? 1 : 2) : phase_of_ins(r - p.n_in);
    return ph == 0 ? src == 0 : ph == 1 ? src == 1 : src >= 1;
  };
  for (int j = 0; j < p.n_ins; j++) {
    const FusedIns &f = p.ins[j];
    if ((f.op == ELT_ROWSUM) != (j == p.sum_ins))
      return 2;
    if (!readable(f.a, j) || !readable(f.op == ELT_ROWSUM ? f.a : f.b, j))
      return 2;
  }
  if (p.out_reg < 0 || p.out_reg >= p.n_in + p.n_ins)
    return 2;
  if (has_sum && phase_of_ins(p.out_reg - p.n_in) != (second_pass ? 2 : 1))
    return 2;
  // merge neighbouring iteration dims that every input walks contiguously (or not at all): fewer divisions per
  // element.  The boundary between rows and the inside of a row is never merged across.
  int64_t dims[ELT_MAX_RANK], str[FUSED_MAX_IN][ELT_MAX_RANK], ostr[ELT_MAX_RANK];
  int nd = 0;
  int64_t inner = 1; // elements of the dims to the right of d
  for (int d = ELT_MAX_RANK - 1; d >= 0; d--) {
    if (p.dims[d] == 1)
      continue;
    bool merge = nd > 0 && !(has_sum && inner == p.n_red);
    for (int k = 0; k < p.n_in && merge; k++)
      merge = p.in_str[k][d] == str[k][nd - 1] * dims[nd - 1];
    if (merge && second_pass)
      merge = p.out_str[d] == ostr[nd - 1] * dims[nd - 1];
    if (merge) {
      dims[nd - 1] *= p.dims[d];
    } else {
      dims[nd] = p.dims[d];
      for (int k = 0; k < p.n_in; k++)
        str[k][nd] = p.in_str[k][d];
      ostr[nd] = p.out_str[d];
      nd++;
    }
    inner *= p.dims[d];
  }
  for (int d = 0; d < ELT_MAX_RANK; d++) {
    const int src = ELT_MAX_RANK - 1 - d; // dims[] was filled innermost first
    p.dims[d] = src < nd ? dims[src] : 1;
    for (int k = 0; k < p.n_in; k++)
      p.in_str[k][d] = src < nd ? str[k][src] : 0;
    p.out_str[d] = src < nd ? ostr[src] : 0;
  }
  p.rank = nd;
  // quad mode: the innermost dim holds whole groups of four, so a thread's four elements share every outer
  // coordinate; an operand contiguous there and aligned (base address and outer strides) moves as one vector
  // (dims are never merged across the boundary of a row, so with a sum the innermost dim lies inside the row
  // whenever the row has more than one element)
  p.quad = nd > 0 && dims[0] % 4 == 0 && (!has_sum || p.n_red > 1) ? 1 : 0;
  p.vec_mask = 0, p.out_vec = 0;
  if (p.quad) {
    auto aligned = [&](const void *ptr, int dt, const int64_t *st_of_dim) {
      const uintptr_t need = dt == PDT_F32 ? 16 : 8;
      if (!assume_aligned && reinterpret_cast<uintptr_t>(ptr) % need != 0)
        return false;
      for (int d = 1; d < nd; d++)
        if (st_of_dim[d] % 4 != 0)
          return false;
      return st_of_dim[0] == 1;
    };
    for (int k = 0; k < p.n_in; k++)
      if (aligned(p.in[k], p.in_dt[k], str[k]))
        p.vec_mask |= 1 << k;
    if (second_pass) {
      p.out_vec = aligned(p.out, p.out_dt, ostr) ? 1 : 0;
    } else {
      const uintptr_t need = p.out_dt == PDT_F32 ? 16 : 8;
      p.out_vec = !has_sum && (assume_aligned || reinterpret_cast<uintptr_t>(p.out) % need == 0) ? 1 : 0;
    }
  }
  // collapsed dims that lie inside a row
  p.rank_red = 0;
  for (int64_t in_row = 1; has_sum && in_row < p.n_red && p.rank_red < nd; p.rank_red++)
    in_row *= dims[p.rank_red];
  return 0;
}

// Register allocation by lifetimes, on a validated program in single-assignment form.  Program order: inputs of a
// phase, then its instructions.  Phases 1 and 3 repeat per element, so a register may be reused inside a phase as
// soon as its value is dead there; a per-row value that the second pass reads stays live to the end.
// Rewrites a, b, out_reg to physical numbers, fills d, in_reg and n_phys; returns n_phys.
inline int fused_allocate(FusedParams &p) {
  const int n_val = p.n_in + p.n_ins;
  const bool has_sum = p.sum_ins >= 0;
  const int row_end = has_sum ? p.row_end : p.n_ins, n_in_pre = has_sum ? p.n_in_pre : p.n_in,
            n_in_row = has_sum ? p.n_in_row : p.n_in;
  auto phase_of_ins = [&](int j) { return !has_sum ? 0 : j < p.sum_ins ? 0 : j < row_end ? 1 : 2; };
  // program points: instruction j sits at 2j+1; the inputs of a phase are defined just before its first instruction
  auto def_point = [&](int v) {
    if (v >= p.n_in)
      return 2 * (v - p.n_in) + 1;
    if (v < n_in_pre)
      return -1;
    return v < n_in_row ? 2 * p.sum_ins + 2 : 2 * row_end;
  };
  const int END = 1 << 20;
  int last[FUSED_MAX_IN + FUSED_MAX_INS];
  for (int v = 0; v < n_val; v++)
    last[v] = def_point(v);
  for (int j = 0; j < p.n_ins; j++) {
    const int srcs[2] = {p.ins[j].a, p.ins[j].op == ELT_ROWSUM ? p.ins[j].a : p.ins[j].b};
    for (int v : srcs) {
      const int def_phase = v < p.n_in ? (v < n_in_pre ? 0 : v < n_in_row ? 1 : 2) : phase_of_ins(v - p.n_in);
      const int use = (has_sum && def_phase == 1 && phase_of_ins(j) == 2) ? END : 2 * j + 1;
      if (use > last[v])
        last[v] = use;
    }
  }
  last[p.out_reg] = END;
  int phys[FUSED_MAX_IN + FUSED_MAX_INS], busy_until[FUSED_MAX_IN + FUSED_MAX_INS];
  for (int r = 0; r < n_val; r++)
    busy_until[r] = -100;
  int n_phys = 0;
  // values in order of definition: inputs of phase 1, its instructions, the sum, inputs of phase 2, ...
  int order[FUSED_MAX_IN + FUSED_MAX_INS], n_order = 0;
  for (int v = 0; v < n_in_pre; v++)
    order[n_order++] = v;
  for (int j = 0; j < p.n_ins; j++) {
    if (has_sum && j == p.sum_ins + 1)
      for (int v = n_in_pre; v < n_in_row; v++)
        order[n_order++] = v;
    if (has_sum && j == row_end)
      for (int v = n_in_row; v < p.n_in; v++)
        order[n_order++] = v;
    order[n_order++] = p.n_in + j;
  }
  if (has_sum && p.sum_ins + 1 >= p.n_ins) // no instruction after the sum: its per-row inputs (none are legal) -- keep order complete
    for (int v = n_in_pre; v < p.n_in; v++)
      order[n_order++] = v;
  for (int q = 0; q < n_order; q++) {
    const int v = order[q], at = def_point(v);
    int r = 0;
    // a source that dies at this instruction frees its register for d (operands are read before d is written)
    while (r < n_val && busy_until[r] > at)
      r++;
    phys[v] = r;
    busy_until[r] = last[v];
    if (r + 1 > n_phys)
      n_phys = r + 1;
  }
  for (int j = 0; j < p.n_ins; j++) {
    p.ins[j].a = phys[p.ins[j].a];
    p.ins[j].b = phys[p.ins[j].b];
    p.ins[j].d = phys[p.n_in + j];
  }
  for (int k = 0; k < p.n_in; k++)
    p.in_reg[k] = phys[k];
  p.out_reg = phys[p.out_reg];
  p.n_phys = n_phys;
  return n_phys;
}

struct SoftmaxParams {
  const void *in;
  void *out;
  int64_t outer, len, inner;
  int32_t in_dt, out_dt;
};

} // namespace gcmi
