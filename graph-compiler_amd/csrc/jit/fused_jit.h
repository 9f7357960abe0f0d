// Run-time specialisation of fused point-wise groups.
//
// The kernels built with the library run a fused group (gcmi::FusedParams) as an interpreter: registers in LDS, one
// dispatch per instruction per step.  That costs a few hundred issue slots per instruction, which is what bounds
// them once the tensors are large.  Here the same program is written out as HIP source for its exact shapes,
// strides, types and ops -- every value a plain float the compiler keeps in a VGPR, every division by a dim a
// constant -- and compiled with hiprtc when the partition is compiled.  This is the part of the reference that a
// JIT serves as well: it lowers each fused group to its own loop nest and compiles it with LLVM
// (lib/gc/Transforms/Pipeline.cpp:105-160, lib/gc/ExecutionEngine/Driver/Driver.cpp:50-77).
//
// The generated kernels evaluate the same expressions in the same order as the interpreter (the op table and the
// rounding helpers are the same source text, kernels/device_math.hpp; the order of the partial sums of a row is the
// interpreter's), with a compiler barrier after every op so that no multiply is contracted into the add of the next
// op: both ways of running a group give the same bits.
#pragma once
#include <hip/hip_runtime_api.h>

#include <memory>
#include <string>
#include <vector>

#include "kernels/eltwise_params.h"

namespace gcjit {

// One generated kernel: its source (a single extern "C" function named `name`) and how to launch it.
struct FusedKernelSource {
  std::string name, source;
  unsigned grid = 0, block = 0;
  int n_in = 0;
  bool quad = false; // moves 16- or 8-byte vectors: every operand address must be 16-byte aligned
};

// Writes the kernel for `p` (pointers are not read: they become kernel arguments in[0] .. in[n_in-1], out).
// same_as[k] = j < k: input k is the same tensor, read through the same strides, as input j (-1: not known to be).
// Returns false when the program is not one the generator covers (the caller keeps the interpreter).
bool generate_fused(const gcmi::FusedParams &p, const int *same_as, const std::string &name, FusedKernelSource &out);

// The kernel for a softmax along the innermost axis of a [rows, len] view (arguments: in0, out).  Returns false for
// rows too long to keep in registers (the library's kernel runs those).
bool generate_softmax(int64_t rows, int64_t len, int in_dt, int out_dt, const std::string &name, FusedKernelSource &out);

// A compiled set of kernels, loaded on the device that was current when it was built.
class Module {
public:
  ~Module();
  hipFunction_t function(const std::string &name) const;
  // Compiles `kernels` as one program for the current device's architecture.  Returns null and sets `error` when
  // the run-time compiler is not available or rejects the source.  Results are cached per process by source text.
  static std::shared_ptr<Module> build(const std::vector<FusedKernelSource> &kernels, std::string &error);
  // The text in front of every generated kernel (type names, op codes, device arithmetic).
  static const char *prelude();

private:
  hipModule_t mod_ = nullptr;
};

// Compiles for `arch` without loading (no GPU needed): the build check of the generator.  Empty string on success,
// the compiler's log otherwise.
std::string compile_only(const std::vector<FusedKernelSource> &kernels, const std::string &arch);

} // namespace gcjit
