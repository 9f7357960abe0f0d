// Host check of gcmi::fused_allocate (kernels/eltwise_params.h): random programs in single-assignment form are
// evaluated as written and again through the physical registers the allocator assigns, phase by phase and with
// the per-element phases repeated, as the kernels run them.  Prints "ok <programs> max <registers>" or a failure.
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>
#include "kernels/eltwise_params.h"
using namespace gcmi;

static uint32_t rng_state = 12345;
static uint32_t rnd(uint32_t n) {
  rng_state = rng_state * 1664525u + 1013904223u;
  return (rng_state >> 8) % n;
}

// value of input k in repetition `rep` of its phase
static double input_value(int k, int rep) { return 1.0 + k * 0.37 + rep * 11.0; }
static double apply(int op, double a, double b) { return op == ELT_ROWSUM ? a * 3.0 + 1.0 : a * 1.25 + b * 0.5 + op; }

int main() {
  int programs = 0, max_regs = 0;
  for (int trial = 0; trial < 20000; trial++) {
    FusedParams p{};
    const bool has_sum = rnd(3) != 0, second = has_sum && rnd(2);
    const int n_pre_in = 1 + rnd(3), n_row_in = has_sum ? rnd(3) : 0, n_p2_in = second ? 1 + rnd(3) : 0;
    p.n_in = n_pre_in + n_row_in + n_p2_in;
    p.n_in_pre = has_sum ? n_pre_in : p.n_in;
    p.n_in_row = has_sum ? n_pre_in + n_row_in : p.n_in;
    const int n_pre = rnd(5), n_row = has_sum ? rnd(4) : 0, n_p2 = second ? 1 + rnd(5) : 0;
    int j = 0;
    std::vector<int> pre_vals, row_vals, p2_vals; // registers readable in each phase
    for (int k = 0; k < n_pre_in; k++)
      pre_vals.push_back(k);
    auto emit = [&](int op, std::vector<int> &pool) {
      p.ins[j].op = op;
      p.ins[j].a = pool[rnd((uint32_t)pool.size())];
      p.ins[j].b = pool[rnd((uint32_t)pool.size())];
      pool.push_back(p.n_in + j);
      j++;
    };
    for (int q = 0; q < n_pre + (has_sum ? 0 : 1); q++)
      emit(ELT_ADD + (int)rnd(3), pre_vals);
    p.sum_ins = -1;
    if (has_sum) {
      p.sum_ins = j;
      p.ins[j].op = ELT_ROWSUM, p.ins[j].a = p.ins[j].b = pre_vals[rnd((uint32_t)pre_vals.size())];
      row_vals.push_back(p.n_in + j);
      j++;
      for (int k = n_pre_in; k < n_pre_in + n_row_in; k++)
        row_vals.push_back(k);
      for (int q = 0; q < n_row; q++)
        emit(ELT_ADD + (int)rnd(3), row_vals);
      p.row_end = j;
      if (second) {
        p2_vals = row_vals;
        for (int k = p.n_in_row; k < p.n_in; k++)
          p2_vals.push_back(k);
        for (int q = 0; q < n_p2; q++)
          emit(ELT_ADD + (int)rnd(3), p2_vals);
      }
    }
    p.n_ins = j;
    if (!has_sum)
      p.row_end = j;
    p.out_reg = p.n_in + j - 1;
    if (p.n_ins > FUSED_MAX_INS || p.n_in > FUSED_MAX_IN)
      continue;
    const FusedParams ssa = p;
    const int n_phys = fused_allocate(p);
    if (n_phys > max_regs)
      max_regs = n_phys;
    programs++;
    // --- as written
    auto phase_of = [&](int jj) { return !has_sum ? 0 : jj < ssa.sum_ins ? 0 : jj < ssa.row_end ? 1 : 2; };
    const int reps = 3;
    std::vector<double> want; // outputs per repetition of the last phase
    {
      std::vector<double> v(ssa.n_in + ssa.n_ins, 0.0);
      for (int rep = 0; rep < reps; rep++) { // phase 0 repeats; the sum sees the last repetition
        for (int k = 0; k < ssa.n_in_pre; k++)
          v[k] = input_value(k, rep);
        for (int jj = 0; jj < ssa.n_ins && phase_of(jj) == 0 && jj != ssa.sum_ins; jj++)
          v[ssa.n_in + jj] = apply(ssa.ins[jj].op, v[ssa.ins[jj].a], v[ssa.ins[jj].b]);
        if (!has_sum)
          want.push_back(v[ssa.out_reg]);
      }
      if (has_sum) {
        v[ssa.n_in + ssa.sum_ins] = apply(ELT_ROWSUM, v[ssa.ins[ssa.sum_ins].a], 0);
        for (int k = ssa.n_in_pre; k < ssa.n_in_row; k++)
          v[k] = input_value(k, 0);
        for (int jj = ssa.sum_ins + 1; jj < ssa.row_end; jj++)
          v[ssa.n_in + jj] = apply(ssa.ins[jj].op, v[ssa.ins[jj].a], v[ssa.ins[jj].b]);
        if (ssa.row_end >= ssa.n_ins)
          want.push_back(v[ssa.out_reg]);
        for (int rep = 0; rep < reps && ssa.row_end < ssa.n_ins; rep++) {
          for (int k = ssa.n_in_row; k < ssa.n_in; k++)
            v[k] = input_value(k, rep);
          for (int jj = ssa.row_end; jj < ssa.n_ins; jj++)
            v[ssa.n_in + jj] = apply(ssa.ins[jj].op, v[ssa.ins[jj].a], v[ssa.ins[jj].b]);
          want.push_back(v[ssa.out_reg]);
        }
      }
    }
    // --- through the physical registers
    std::vector<double> got;
    {
      std::vector<double> r((size_t)n_phys + 1, -777.0);
      auto run = [&](int j0, int j1) {
        for (int jj = j0; jj < j1; jj++) {
          const double a = r[p.ins[jj].a], b = r[p.ins[jj].b];
          r[p.ins[jj].d] = apply(p.ins[jj].op, a, b);
        }
      };
      const int pre_end = has_sum ? p.sum_ins : p.n_ins;
      for (int rep = 0; rep < reps; rep++) {
        for (int k = 0; k < p.n_in_pre; k++)
          r[p.in_reg[k]] = input_value(k, rep);
        run(0, pre_end);
        if (!has_sum)
          got.push_back(r[p.out_reg]);
      }
      if (has_sum) {
        r[p.ins[p.sum_ins].d] = apply(ELT_ROWSUM, r[p.ins[p.sum_ins].a], 0);
        for (int k = p.n_in_pre; k < p.n_in_row; k++)
          r[p.in_reg[k]] = input_value(k, 0);
        run(p.sum_ins + 1, p.row_end);
        if (p.row_end >= p.n_ins)
          got.push_back(r[p.out_reg]);
        for (int rep = 0; rep < reps && p.row_end < p.n_ins; rep++) {
          for (int k = p.n_in_row; k < p.n_in; k++)
            r[p.in_reg[k]] = input_value(k, rep);
          run(p.row_end, p.n_ins);
          got.push_back(r[p.out_reg]);
        }
      }
    }
    if (want.size() != got.size() || memcmp(want.data(), got.data(), want.size() * sizeof(double)) != 0) {
      printf("mismatch in trial %d (n_in %d n_ins %d sum %d row_end %d regs %d)\n", trial, ssa.n_in, ssa.n_ins,
             ssa.sum_ins, ssa.row_end, n_phys);
      return 1;
    }
  }
  printf("ok %d max %d\n", programs, max_regs);
  return 0;
}
