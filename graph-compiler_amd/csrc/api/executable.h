// A compiled partition: a list of kernel launches over device buffers.
//
// compile  = parse (graph.h) -> verify -> fuse -> plan.  Fusion replaces the
//            reference's tiling + consumer fusion passes
//            (lib/gc/Transforms/DeepTileContractionOp.cpp,
//             lib/gc/Transforms/IterativeTilingAndFusion.cpp:585-611): a MatMul
//            absorbs the bias add / activation / cast that follow it into the
//            GEMM epilogue; Dequantize -> MatMul becomes the int8 GEMM with a
//            dequantising epilogue; MatMul -> scale -> +mask -> SoftMax ->
//            MatMul becomes one attention kernel.  Everything else runs as a
//            generic kernel per op.
// execute  = match tensors by id (src/dnnl/dnnl_graph_compiler.cpp:64-103),
//            stage host buffers to the device arena (device pointers are used
//            in place), launch, copy results back, wait.
#pragma once
#include <hip/hip_runtime_api.h>

#include <cstdint>
#include <map>
#include <mutex>
#include <string>
#include <unordered_map>
#include <vector>

#include "dnnl_graph_compiler.h"
#include "graph.h"
#include "jit/fused_jit.h"

namespace gcapi {

struct Step {
  enum Kind { GemmF32, GemmBf16, GemmInt8, ColSum, Mha, Elt, Reduce, Softmax, Fused, MhaClassify } kind;
  std::string note; // what was fused, for introspection
  bool once = false; // depends on constant tensors only: runs in the first execute, its result is kept
  // operands are arena slot indices (-1 = none)
  int a = -1, b = -1, c = -1, out = -1, bias = -1, mask = -1, aux = -1;
  // the op's MatmulConfig attributes {MThreads, NThreads, KThreads, MBlock, NBlock, KBlock, innermostMBlock,
  // innermostNBlock, innermostKBlock} when all nine are there (lib/gc/Analysis/MatmulConfigAnalysis.cpp:368-404)
  std::vector<int64_t> mm_cfg;
  int ws = -1; // scratch of this step alone (partial sums of a K-sliced GEMM, mask tile classes of attention)
  int64_t M = 0, N = 0, K = 0, lda = 0, ldb = 0, ldc = 0;
  int64_t a_off = 0, b_off = 0, out_off = 0; // element offsets (batched fallbacks)
  int64_t batch = 1, a_bs = 0, b_bs = 0, c_bs = 0; // strided batch in one launch (0 stride: shared operand)
  bool ta = false, tb = false;
  int act = 0, out_dt = 0, bias_dt = 0, a_dt = 0;
  int32_t zp = 0;
  // attention
  int64_t BH = 0, Sq = 0, Sk = 0, D = 0, mask_ld = 0;
  float scale = 1.0f;
  int scale_slot = -1;   // 1-element tensor holding the scale (or its reciprocal)
  bool scale_div = false;
  bool classes_valid = false; // `ws` holds the mask's tile classes, prepared by a once-only MhaClassify step
  // generic kernels: parameter blocks are filled at plan time with slot ids
  // resolved to pointers at execute time
  std::vector<int64_t> dims, sa, sb;
  int op = 0, b_dt = 0;
  float alpha = 0;
  int n_scales = 0, ch_axis = -1, scales_slot = -1, zps_slot = -1;
  // reduce
  std::vector<int64_t> kdims, kstr, rdims, rstr;
  bool mean = false;
  // softmax
  int64_t outer = 0, len = 0, inner = 0;
  // fused point-wise group (gcmi::FusedParams): inputs with their strides over `dims`, the program, and for a
  // group that feeds a sum the row length and the register that is summed
  struct FIns {
    int op, a, b, dt;
    float imm;
  };
  std::vector<int> f_in, f_in_dt;
  std::vector<std::vector<int64_t>> f_str;
  std::vector<FIns> f_ins;
  int64_t n_red = 0;
  int red_reg = 0; // the register that is stored
  int n_in_pre = 0, sum_ins = -1;
  int n_in_row = -1, row_end = -1;   // second pass of a row kernel (-1: none)
  std::vector<int64_t> out_str;      // its output strides over `dims`
  // planning only: what the group holds (ops, the tensor behind each input, the tensor it writes) and, for a
  // group with a sum, where each non-unit dim of the full shape sits in `dims`
  std::vector<size_t> f_members, f_in_tensor;
  size_t f_out_tensor = 0;
  std::vector<int> f_place;
  // the kernel generated for this group when the partition was compiled (null: the library's interpreter runs it)
  hipFunction_t jit_fn = nullptr;
  unsigned jit_grid = 0, jit_block = 0;
  bool jit_vectors = false; // it moves 16-byte vectors: the operands must be aligned
};

struct Slot {
  size_t bytes = 0;
  size_t offset = 0;   // into the arena, or into the staging block when `staged`
  bool staged = false; // a graph input / output that the caller's device pointer replaces: no arena space (executable.cpp, layout_arena)
  long tensor_id = -1; // graph tensor it holds, -1 for temporaries / constants
  bool is_input = false, is_output = false;
  std::vector<char> init; // constant contents uploaded at compile time
};

class Executable {
public:
  // dry = plan only: no device memory, no stream (host-side tests and explain)
  explicit Executable(const char *json, bool dry = false);
  // from a graph built by another front end (mlir_text.h)
  explicit Executable(Graph g, bool dry = false);
  ~Executable();
  Executable(const Executable &) = delete;
  Executable &operator=(const Executable &) = delete;

  void execute(dnnl_graph_compiler_tensor *inputs, dnnl_graph_compiler_tensor *outputs);
  // the same launches on the caller's stream, without waiting for them: device pointers only
  void execute_async(dnnl_graph_compiler_tensor *inputs, dnnl_graph_compiler_tensor *outputs, hipStream_t stream);

  const Graph &graph() const { return g_; }
  const std::vector<Step> &steps() const { return steps_; }
  std::string describe() const; // one line per step
  // HIP source of the kernels that are generated for the fused groups of this plan (dry plans included)
  std::vector<gcjit::FusedKernelSource> generated_kernels() const;
  // launches of generated kernels by all executables of the process (tests check that the generated path ran)
  static long generated_launches();

private:
  Graph g_;
  std::vector<Step> steps_;
  std::vector<Slot> slots_;
  std::unordered_map<size_t, int> slot_of_tensor_;
  std::vector<void *> ptr_; // per-slot device pointer during execute (guarded by run_mu_)
  // execute() may be called from several host threads (the reference's execute is const and re-entrant,
  // src/dnnl/dnnl_graph_compiler.cpp:214-226): calls on one executable take turns, since they share its arena
  std::mutex run_mu_;
  // results of once-only steps: computed on the stream of the first call, waited for by calls on other streams
  hipEvent_t once_done_ = nullptr;
  hipStream_t once_stream_ = nullptr;
  bool once_recorded_ = false;
  char *arena_ = nullptr;
  size_t arena_bytes_ = 0;
  size_t arena_bytes_no_reuse_ = 0; // what one region per slot would take
  // device copies of the caller's HOST buffers (graph inputs and outputs): one block, allocated by the first
  // execute that passes a host pointer -- a caller that keeps its tensors on the device never pays for it
  char *staging_ = nullptr;
  size_t staging_bytes_ = 0;
  char *staging();
  void release() noexcept;
  hipStream_t stream_ = nullptr;
  std::unordered_map<int, bool> colsum_valid_; // ColSum results of constant weights are computed once
  std::vector<char> step_done_;                // per step: a `once` step has run
  std::vector<char> const_staged_;             // per slot: a constant host input has been copied to the device
  std::shared_ptr<gcjit::Module> jit_module_;  // the generated kernels of the fused groups

  int new_slot(size_t bytes, long tensor_id = -1);
  int slot_for(size_t tensor_id);
  int const_slot(const void *data, size_t bytes);
  void init(bool dry);
  void plan();
  void plan_workspaces();
  void layout_arena();
  void plan_generic(const Op &op);
  void plan_fusion(std::vector<bool> &skip, const std::vector<bool> &claimed, std::map<size_t, std::vector<Step>> &emit_at,
                   bool groups);
  void plan_matmul(size_t op_index, std::vector<bool> &done);
  bool try_int8(size_t op_index, std::vector<bool> &done);
  bool try_mha(size_t op_index, std::vector<bool> &done);
  void add_copy(int src_slot, DT src_dt, const std::vector<int64_t> &dims, const std::vector<int64_t> &strides,
                int dst_slot, DT dst_dt);
  void launch(const Step &s);
  void run(dnnl_graph_compiler_tensor *inputs, dnnl_graph_compiler_tensor *outputs, bool wait);
  void build_generated_kernels();
};

} // namespace gcapi
