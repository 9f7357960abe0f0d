#include "executable.h"

#include <algorithm>
#include <atomic>
#include <cmath>
#include <cstdlib>
#include <cstring>
#include <map>
#include <set>
#include <sstream>
#include <stdexcept>

#include "gc_hip_kernels.h"
#include "kernels/eltwise_params.h"

extern "C" {
int gcmi_launch_eltwise(const gcmi::EltParams *p, hipStream_t stream);
int gcmi_launch_reduce(const gcmi::ReduceParams *p, hipStream_t stream);
int gcmi_launch_fused(const gcmi::FusedParams *p, hipStream_t stream);
int gcmi_launch_softmax(const gcmi::SoftmaxParams *p, hipStream_t stream);
}

namespace gcapi {

namespace {

void hip_check(hipError_t e, const char *what) {
  if (e != hipSuccess) {
    if (e == hipErrorOutOfMemory)
      throw std::bad_alloc();
    throw std::runtime_error(std::string(what) + ": " + hipGetErrorString(e));
  }
}
void gc_check(int rc, const char *what) {
  if (rc != 0)
    throw std::runtime_error(std::string(what) + ": " + gcmi_last_error());
}

// IEEE binary16 bits of x, round to nearest even (the host compiler has no half type)
static uint16_t f32_to_f16_bits(float x) {
  uint32_t u;
  memcpy(&u, &x, 4);
  const uint32_t sign = (u >> 16) & 0x8000u;
  u &= 0x7fffffffu;
  if (u >= 0x7f800000u) // inf / nan
    return (uint16_t)(sign | 0x7c00u | (u > 0x7f800000u ? 0x200u : 0));
  if (u >= 0x477ff000u) // rounds to 65520 or more: inf
    return (uint16_t)(sign | 0x7c00u);
  if (u < 0x38800000u) { // below the smallest normal half: fixed point with 24 fraction bits
    if (u < 0x33000000u)
      return (uint16_t)sign; // under half of the smallest subnormal
    const int shift = 126 - (int)(u >> 23); // 14 .. 24
    const uint32_t mant = (u & 0x7fffffu) | 0x800000u;
    const uint32_t q = mant >> shift, rem = mant & ((1u << shift) - 1), half = 1u << (shift - 1);
    return (uint16_t)(sign | (q + (rem > half || (rem == half && (q & 1)))));
  }
  const uint32_t e = (u >> 23) - 112, m = u & 0x7fffffu;
  uint32_t h = (e << 10) | (m >> 13);
  const uint32_t rem = m & 0x1fffu;
  h += rem > 0x1000u || (rem == 0x1000u && (h & 1));
  return (uint16_t)(sign | h);
}

std::vector<int64_t> dense_strides(const std::vector<int64_t> &shape) {
  std::vector<int64_t> s(shape.size(), 1);
  for (int i = (int)shape.size() - 2; i >= 0; i--)
    s[i] = s[i + 1] * shape[i + 1];
  return s;
}
bool is_dense(const LTensor &t) { return !t.strided || t.stride == dense_strides(t.shape); }
int64_t prod(const std::vector<int64_t> &v, size_t lo, size_t hi) {
  int64_t p = 1;
  for (size_t i = lo; i < hi; i++)
    p *= v[i];
  return p;
}
bool is_device_pointer(const void *p) {
  hipPointerAttribute_t attr;
  hipError_t e = hipPointerGetAttributes(&attr, p);
  if (e != hipSuccess) {
    (void)hipGetLastError(); // plain host memory is reported as an error: clear it
    return false;
  }
  return attr.type == hipMemoryTypeDevice;
}
size_t align256(size_t v) { return (v + 255) & ~(size_t)255; }

int act_of(const Op &op) {
  if (op.kind == "ReLU")
    return GCMI_ACT_RELU;
  if (op.kind == "Sigmoid")
    return GCMI_ACT_SIGMOID;
  if (op.kind == "GELU") {
    std::string m = op.attr_str("mode", "gelu_erf");
    if (m == "gelu_tanh" || m == "tanh")
      return GCMI_ACT_GELU_TANH;
    if (m == "gelu_erf" || m == "erf")
      return GCMI_ACT_GELU_ERF;
    throw std::logic_error("Unsupported GELU mode: " + m);
  }
  return -1;
}

// [N] or [1,..,1,N]
bool is_row_vector(const LTensor &t, int64_t N) {
  if (t.shape.empty() || t.shape.back() != N)
    return false;
  for (size_t i = 0; i + 1 < t.shape.size(); i++)
    if (t.shape[i] != 1)
      return false;
  return true;
}

} // namespace

// ---------------------------------------------------------------------------
int Executable::new_slot(size_t bytes, long tensor_id) {
  Slot s;
  s.bytes = bytes ? bytes : 4;
  s.tensor_id = tensor_id;
  slots_.push_back(std::move(s));
  return (int)slots_.size() - 1;
}

int Executable::slot_for(size_t tid) {
  auto it = slot_of_tensor_.find(tid);
  if (it != slot_of_tensor_.end())
    return it->second;
  const LTensor &t = g_.tensors.at(tid);
  int es = dt_size(t.dt);
  if (es == 0)
    throw std::logic_error(std::string("Unsupported tensor dtype on this path: ") + dt_name(t.dt));
  if (t.alias_of >= 0) { // a reshape view: the storage of the tensor it views
    int s = slot_for((size_t)t.alias_of);
    slot_of_tensor_[tid] = s;
    return s;
  }
  if (t.has_splat) { // one element, read with stride 0
    uint32_t bits = 0;
    float f = (float)t.splat;
    if (t.dt == DT::f32)
      memcpy(&bits, &f, 4);
    else if (t.dt == DT::bf16) {
      uint32_t u;
      memcpy(&u, &f, 4);
      bits = (u + 0x7FFFu + ((u >> 16) & 1u)) >> 16;
    } else if (t.dt == DT::f16) {
      bits = f32_to_f16_bits(f);
    } else
      throw std::logic_error(std::string("Constant of this dtype is not supported: ") + dt_name(t.dt));
    int s = const_slot(&bits, (size_t)es);
    slot_of_tensor_[tid] = s;
    return s;
  }
  int s = new_slot((size_t)t.numel() * es, (long)tid);
  slot_of_tensor_[tid] = s;
  return s;
}

int Executable::const_slot(const void *data, size_t bytes) {
  int s = new_slot(bytes);
  slots_[s].init.assign((const char *)data, (const char *)data + bytes);
  return s;
}

void Executable::add_copy(int src, DT sdt, const std::vector<int64_t> &dims, const std::vector<int64_t> &strides,
                          int dst, DT ddt) {
  if (dims.size() > (size_t)gcmi::ELT_MAX_RANK)
    throw std::logic_error("tensor rank above 6 is not supported");
  Step s;
  s.kind = Step::Elt;
  s.note = "copy";
  s.op = gcmi::ELT_COPY;
  s.a = src, s.out = dst;
  s.a_dt = dt_dnnl(sdt), s.out_dt = dt_dnnl(ddt);
  s.dims = dims, s.sa = strides;
  steps_.push_back(std::move(s));
}

// The nine MatmulConfig attributes of a matmul op, in the order the kernels' ABI takes them; empty unless all nine
// are integer attributes (the reference uses a config only when it is complete, MatmulConfigAnalysis.cpp:368-404).
static std::vector<int64_t> matmul_config_attrs(const Op &op) {
  static const char *names[9] = {"MThreads", "NThreads", "KThreads", "MBlock", "NBlock", "KBlock",
                                 "innermostMBlock", "innermostNBlock", "innermostKBlock"};
  std::vector<int64_t> v;
  for (const char *n : names) {
    auto it = op.attrs.find(n);
    if (it == op.attrs.end() || it->second.type != Attr::S64)
      return {};
    v.push_back(it->second.i);
  }
  return v;
}

// ---------------------------------------------------------------------------
Executable::Executable(const char *json, bool dry) : g_(parse_graph(json)) { init(dry); }
Executable::Executable(Graph g, bool dry) : g_(std::move(g)) { init(dry); }

void Executable::init(bool dry) {
  verify_graph(g_);
  plan();
  plan_workspaces();
  layout_arena();
  if (dry)
    return;
  try { // a constructor that throws runs no destructor: what has been acquired is given back here
    hip_check(hipMalloc((void **)&arena_, arena_bytes_), "hipMalloc(arena)");
    hip_check(hipStreamCreate(&stream_), "hipStreamCreate");
    for (auto &s : slots_)
      if (!s.init.empty())
        hip_check(hipMemcpy(arena_ + s.offset, s.init.data(), s.init.size(), hipMemcpyHostToDevice), "upload constants");
    ptr_.resize(slots_.size());
    build_generated_kernels();
  } catch (...) {
    release();
    throw;
  }
}

void Executable::release() noexcept {
  if (once_done_)
    (void)hipEventDestroy(once_done_);
  if (stream_)
    (void)hipStreamDestroy(stream_);
  if (arena_)
    (void)hipFree(arena_);
  if (staging_)
    (void)hipFree(staging_);
  once_done_ = nullptr, stream_ = nullptr, arena_ = nullptr, staging_ = nullptr;
}

char *Executable::staging() {
  if (!staging_)
    hip_check(hipMalloc((void **)&staging_, staging_bytes_ ? staging_bytes_ : 256), "hipMalloc(staging for host buffers)");
  return staging_;
}

// Scratch of the steps whose kernels need some (partial sums of K-sliced GEMMs, mask tile classes of attention): a
// slot of the step's own, alive for that step only, so it shares arena space with other temporaries.  Nothing is
// shared between executables or streams: two executables may run side by side, as the reference's may
// (thread-local scratch, lib/gc/ExecutionEngine/CPURuntime/Microkernel/BrgemmOnednn.cpp:70).
void Executable::plan_workspaces() {
  for (Step &s : steps_) {
    size_t bytes = 0;
    if (s.kind == Step::GemmBf16 && s.batch <= 1)
      bytes = gcmi_gemm_bf16_workspace_bytes_cfg(s.M, s.N, s.K, s.tb ? 1 : 0, s.mm_cfg.size() == 9 ? s.mm_cfg.data() : nullptr);
    else if (s.kind == Step::Mha && s.mask >= 0 && s.ws < 0)
      bytes = gcmi_mha_fwd_workspace_bytes(s.Sq, s.Sk, s.D, 1);
    if (bytes)
      s.ws = new_slot(bytes);
  }
}

// One allocation per executable, temporaries with disjoint lifetimes share memory: the tick-based merge
// of the reference (lib/gc/Transforms/MergeAllocTickBased.cpp, docs/memref_schedule.md) with the step
// index as the tick.  A slot lives from the first step that names it to the last; graph inputs and
// outputs, constants and the results of once-only steps live for the whole executable.  Temporaries
// are placed in order of their first tick at the lowest offset that is free for their whole lifetime.
void Executable::layout_arena() {
  const int n = (int)slots_.size();
  std::vector<int> first(n, -1), last(n, -1);
  std::vector<char> pinned(n, 0);
  auto touch = [&](int slot, int tick) {
    if (slot < 0)
      return;
    if (first[slot] < 0)
      first[slot] = tick;
    last[slot] = tick;
  };
  for (int i = 0; i < (int)steps_.size(); i++) {
    const Step &s = steps_[i];
    for (int slot : {s.a, s.b, s.c, s.out, s.bias, s.mask, s.aux, s.ws, s.scale_slot, s.scales_slot, s.zps_slot})
      touch(slot, i);
    for (int slot : s.f_in)
      touch(slot, i);
    if (s.once || (s.kind == Step::ColSum && s.op == 1))
      if (s.out >= 0)
        pinned[s.out] = 1;
  }
  // Graph inputs and outputs are the caller's buffers: a device pointer is used in place, and only a host buffer
  // needs a device copy -- those copies live in a block of their own that the first such execute allocates.
  // (An output that a once-only step computes stays in the arena: it is written once and copied out per call.)
  size_t stage_off = 0;
  for (int i = 0; i < n; i++) {
    Slot &sl = slots_[i];
    sl.staged = (sl.is_input || sl.is_output) && sl.init.empty() && !pinned[i];
    if (sl.staged) {
      sl.offset = stage_off;
      stage_off += align256(sl.bytes);
    } else if (sl.is_input || sl.is_output || !sl.init.empty() || first[i] < 0) {
      pinned[i] = 1;
    }
  }
  staging_bytes_ = stage_off;
  size_t off = 0, naive = 0;
  for (int i = 0; i < n; i++) {
    if (slots_[i].staged)
      continue;
    naive += align256(slots_[i].bytes);
    if (pinned[i]) {
      slots_[i].offset = off;
      off += align256(slots_[i].bytes);
    }
  }
  const size_t temp_base = off;
  std::vector<int> order;
  for (int i = 0; i < n; i++)
    if (!pinned[i] && !slots_[i].staged)
      order.push_back(i);
  std::stable_sort(order.begin(), order.end(), [&](int x, int y) { return first[x] < first[y]; });
  std::vector<int> placed;
  size_t top = temp_base;
  for (int i : order) {
    // regions of already placed temporaries whose lifetimes overlap this one, by offset
    std::vector<std::pair<size_t, size_t>> busy;
    for (int j : placed)
      if (!(last[j] < first[i] || last[i] < first[j]))
        busy.emplace_back(slots_[j].offset, slots_[j].offset + align256(slots_[j].bytes));
    std::sort(busy.begin(), busy.end());
    size_t at = temp_base;
    const size_t need = align256(slots_[i].bytes);
    for (auto &b : busy) {
      if (at + need <= b.first)
        break;
      at = std::max(at, b.second);
    }
    slots_[i].offset = at;
    top = std::max(top, at + need);
    placed.push_back(i);
  }
  arena_bytes_ = top ? top : 256;
  arena_bytes_no_reuse_ = naive ? naive : 256;
}

Executable::~Executable() { release(); }

// ---------------------------------------------------------------------------
void Executable::plan() {
  const size_t n = g_.ops.size();
  std::map<size_t, std::vector<size_t>> consumers;
  for (size_t i = 0; i < n; i++)
    for (auto id : g_.ops[i].in)
      consumers[id].push_back(i);
  std::set<size_t> outs(g_.output_ids.begin(), g_.output_ids.end());
  std::map<size_t, size_t> producer;
  for (size_t i = 0; i < n; i++)
    for (auto id : g_.ops[i].out)
      producer[id] = i;

  // strided (non-dense) inputs are gathered into dense buffers first
  for (auto id : g_.input_ids) {
    const LTensor &t = g_.tensors.at(id);
    if (!is_dense(t)) {
      int64_t span = 1;
      for (size_t d = 0; d < t.shape.size(); d++) {
        if (t.stride[d] < 0)
          throw std::logic_error("negative strides are not supported");
        span += (t.shape[d] - 1) * t.stride[d];
      }
      int raw = new_slot((size_t)span * dt_size(t.dt));
      slots_[raw].is_input = true;
      slots_[raw].tensor_id = (long)id;
      int dense = new_slot((size_t)t.numel() * dt_size(t.dt));
      slot_of_tensor_[id] = dense;
      add_copy(raw, t.dt, t.shape, t.stride, dense, t.dt);
    } else {
      slots_[slot_for(id)].is_input = true;
    }
  }
  for (auto id : g_.output_ids) {
    const LTensor &t = g_.tensors.at(id);
    if (!is_dense(t))
      throw std::logic_error("strided output tensors are not supported");
    slots_[slot_for(id)].is_output = true;
  }

  // ---- matching pass: fused groups are emitted where their LAST op stands
  std::vector<bool> skip(n, false), claimed(n, false);
  std::map<size_t, std::vector<Step>> emit_at;
  auto single_use = [&](size_t tid) { return !outs.count(tid) && consumers[tid].size() == 1; };

  for (size_t i = 0; i < n; i++) {
    const Op &mm = g_.ops[i];
    if (mm.kind != "MatMul" || claimed[i])
      continue;
    auto T = [&](size_t id) -> const LTensor & { return g_.tensors.at(id); };
    const bool ta = mm.attr_bool("transpose_a", false), tb = mm.attr_bool("transpose_b", false);

    // ---------------- attention: MatMul(Q,K^T) -> [scale] -> [+mask] -> SoftMax -> MatMul(P,V)
    {
      const LTensor &q = T(mm.in[0]), &k = T(mm.in[1]);
      size_t r = q.shape.size();
      bool ok = mm.in.size() == 2 && !ta && tb && q.dt == DT::bf16 && k.dt == DT::bf16 && r >= 3 &&
                k.shape.size() == r && (q.shape[r - 1] == 128 || q.shape[r - 1] == 64) &&
                std::equal(q.shape.begin(), q.shape.end() - 2, k.shape.begin());
      size_t cur = mm.out[0];
      std::vector<size_t> chain{i};
      long scale_t = -1, mask_t = -1;
      bool scale_div = false;
      size_t last = i;
      if (ok) {
        int64_t Sq = q.shape[r - 2], Sk = k.shape[r - 2];
        bool seen_softmax = false;
        while (ok) {
          if (!single_use(cur)) {
            ok = false;
            break;
          }
          size_t ci = consumers[cur][0];
          const Op &c = g_.ops[ci];
          if ((c.kind == "Multiply" || c.kind == "Divide") && scale_t < 0 && mask_t < 0) {
            size_t other = c.in[0] == cur ? c.in[1] : c.in[0];
            if (c.kind == "Divide" && c.in[0] != cur) {
              ok = false;
              break;
            }
            const LTensor &st = T(other);
            bool is_in = std::find(g_.input_ids.begin(), g_.input_ids.end(), other) != g_.input_ids.end();
            // a one-element input tensor, or a constant of one repeated value (MLIR's dense<x> splat)
            bool one_input = st.numel() == 1 && is_in && (st.dt == DT::f32 || st.dt == DT::bf16);
            if (!one_input && !st.has_splat) {
              ok = false;
              break;
            }
            scale_t = (long)other, scale_div = c.kind == "Divide";
          } else if (c.kind == "Add" && mask_t < 0) {
            size_t other = c.in[0] == cur ? c.in[1] : c.in[0];
            const LTensor &mt = T(other);
            size_t mr = mt.shape.size();
            bool shape_ok = mr >= 2 && mt.shape[mr - 1] == Sk && mt.shape[mr - 2] == Sq && prod(mt.shape, 0, mr - 2) == 1;
            if (!shape_ok || !(mt.dt == DT::f32 || mt.dt == DT::bf16) ) {
              ok = false;
              break;
            }
            mask_t = (long)other;
          } else if (c.kind == "SoftMax") {
            int64_t ax = c.attr_s64("axis", 1);
            if (ax < 0)
              ax += (int64_t)r;
            if (ax != (int64_t)r - 1) {
              ok = false;
              break;
            }
            seen_softmax = true;
          } else if (c.kind == "MatMul" && seen_softmax) {
            const LTensor &v = T(c.in[1]);
            bool fin = c.in.size() == 2 && c.in[0] == cur && !c.attr_bool("transpose_a", false) &&
                       !c.attr_bool("transpose_b", false) && v.dt == DT::bf16 && v.shape.size() == r &&
                       v.shape[r - 1] == q.shape[r - 1] && v.shape[r - 2] == Sk &&
                       std::equal(q.shape.begin(), q.shape.end() - 2, v.shape.begin()) && T(c.out[0]).dt == DT::bf16;
            if (!fin) {
              ok = false;
              break;
            }
            chain.push_back(ci);
            last = ci;
            break;
          } else {
            ok = false;
            break;
          }
          if (seen_softmax && c.kind != "SoftMax") {
            ok = false;
            break;
          }
          chain.push_back(ci);
          cur = c.out[0];
        }
        if (ok && last != i) {
          const Op &pv = g_.ops[last];
          std::vector<Step> v;
          int mask_slot = -1;
          int64_t mask_ld = 0;
          if (mask_t >= 0) {
            const LTensor &mt = T((size_t)mask_t);
            mask_slot = slot_for((size_t)mask_t);
            mask_ld = Sk;
            if (mt.dt != DT::f32) { // the kernel adds an f32 mask
              int f = new_slot((size_t)mt.numel() * 4);
              Step cp;
              cp.kind = Step::Elt, cp.note = mt.constant ? "mask -> f32, once: the mask is constant" : "mask -> f32";
              cp.once = mt.constant, cp.op = gcmi::ELT_COPY, cp.a = mask_slot, cp.out = f;
              cp.a_dt = dt_dnnl(mt.dt), cp.out_dt = GCMI_F32;
              cp.dims = {mt.numel()}, cp.sa = {1};
              v.push_back(cp);
              mask_slot = f;
            }
          }
          Step s;
          s.kind = Step::Mha;
          s.note = "attention: MatMul+scale+mask+SoftMax+MatMul fused (" + std::to_string(chain.size()) + " ops)";
          s.a = slot_for(mm.in[0]), s.b = slot_for(mm.in[1]), s.c = slot_for(pv.in[1]), s.out = slot_for(pv.out[0]);
          s.mask = mask_slot, s.mask_ld = mask_ld;
          s.BH = prod(q.shape, 0, r - 2), s.Sq = Sq, s.Sk = Sk, s.D = q.shape[r - 1];
          if (mask_t >= 0 && T((size_t)mask_t).constant) {
            // A constant mask is classified once per executable (its tiles: all 0, all -inf, general), like the column
            // sums of constant weights: the reference's constant-tensor cache (src/dnnl/JsonParser.cpp:295-299).
            const size_t bytes = gcmi_mha_fwd_workspace_bytes(Sq, Sk, s.D, 1);
            if (bytes) {
              Step cl;
              cl.kind = Step::MhaClassify, cl.note = "mask tile classes, once: the mask is constant", cl.once = true;
              cl.a = mask_slot, cl.mask_ld = mask_ld, cl.Sq = Sq, cl.Sk = Sk, cl.D = s.D;
              cl.out = new_slot(bytes);
              v.push_back(cl);
              s.ws = cl.out, s.classes_valid = true;
            }
          }
          s.scale = 1.0f;
          if (scale_t >= 0 && T((size_t)scale_t).has_splat) {
            const float x = (float)T((size_t)scale_t).splat;
            s.scale = scale_div ? 1.0f / x : x;
          } else if (scale_t >= 0) {
            s.scale_slot = slot_for((size_t)scale_t);
            s.scale_div = scale_div;
            s.a_dt = dt_dnnl(T((size_t)scale_t).dt);
          }
          v.push_back(s);
          for (auto ci : chain)
            skip[ci] = claimed[ci] = true;
          skip[last] = false;
          emit_at[last] = v;
          continue;
        }
      }
    }

    // ---------------- quantised: Dequantize(A) , Dequantize(W) -> MatMul -> [bias] -> [act] -> [cast]
    bool int8 = false;
    size_t dq_a = 0, dq_w = 0;
    if (!ta && producer.count(mm.in[0]) && producer.count(mm.in[1]) && T(mm.out[0]).dt == DT::f32) {
      dq_a = producer[mm.in[0]], dq_w = producer[mm.in[1]];
      const Op &da = g_.ops[dq_a], &dw = g_.ops[dq_w];
      if (da.kind == "Dequantize" && dw.kind == "Dequantize" && single_use(mm.in[0]) && single_use(mm.in[1])) {
        const LTensor &qa = T(da.in[0]), &qw = T(dw.in[0]);
        const auto &sa = da.attrs.at("scales").fa, &sw = dw.attrs.at("scales").fa;
        std::vector<int64_t> zw;
        if (dw.attrs.count("zps"))
          zw = dw.attrs.at("zps").ia;
        bool zw0 = std::all_of(zw.begin(), zw.end(), [](int64_t z) { return z == 0; });
        int64_t axw = dw.attr_s64("axis", 1);
        if (axw < 0)
          axw += (int64_t)qw.shape.size();
        int8 = sa.size() == 1 && qw.dt == DT::s8 && qw.shape.size() == 2 && qa.shape.size() >= 2 && zw0 &&
               (sw.size() == 1 || axw == (tb ? 0 : 1)) && is_dense(qa) && is_dense(qw); // scales per output channel
      }
    }

    // ---------------- epilogue chain shared by the plain and the quantised GEMM
    const LTensor &A = T(mm.in[0]), &B = T(mm.in[1]);
    const size_t ra = A.shape.size(), rb = B.shape.size();
    // fusable only when the contraction is one flat GEMM: [.., M, K] x [K, N]
    bool flat = ra >= 2 && rb == 2 && (!ta || ra == 2);
    int64_t Nn = flat ? (tb ? B.shape[0] : B.shape[1]) : 0;
    long bias_t = mm.in.size() == 3 ? (long)mm.in[2] : -1;
    bool bias_in_matmul = bias_t >= 0;
    if (bias_t >= 0 && !(flat && is_row_vector(T((size_t)bias_t), Nn)))
      bias_t = -1; // handled as a separate Add below
    int act = 0;
    long res_t = -1; // a tensor of the result's shape that is added last (a residual connection): bf16 GEMMs
    size_t cur = mm.out[0], last = i;
    std::vector<size_t> chain;
    DT gemm_dt = int8 ? DT::f32 : A.dt;
    if (flat && (gemm_dt == DT::f32 || gemm_dt == DT::bf16) && (bias_in_matmul ? bias_t >= 0 : true)) {
      while (single_use(cur) && res_t < 0) {
        size_t ci = consumers[cur][0];
        const Op &c = g_.ops[ci];
        if (claimed[ci])
          break;
        if (c.kind == "Add") {
          size_t other = c.in[0] == cur ? c.in[1] : c.in[0];
          const LTensor &bt = T(other);
          bool dt_ok = bt.dt == T(cur).dt;
          if (!dt_ok || T(c.out[0]).shape != T(cur).shape)
            break;
          if (bias_t < 0 && act == 0 && is_row_vector(bt, Nn))
            bias_t = (long)other;
          else if (!int8 && gemm_dt == DT::bf16 && bt.shape == T(cur).shape && !bt.has_splat)
            res_t = (long)other;
          else
            break;
        } else if (c.kind == "Reshape" && T(c.out[0]).alias_of >= 0 && !T(c.out[0]).shape.empty() &&
                   T(c.out[0]).shape.back() == Nn) {
          // a view of the result that keeps its rows (tensor.expand_shape to [1, M, N] and the like): the ops
          // behind it fuse as they would without it
        } else if (act_of(c) > 0 && act == 0) {
          act = act_of(c);
        } else if (int8 && (c.kind == "Typecast" || c.kind == "TypeCast") && T(c.out[0]).dt == DT::bf16) {
          chain.push_back(ci);
          last = ci;
          cur = c.out[0];
          break;
        } else {
          break;
        }
        chain.push_back(ci);
        last = ci;
        cur = c.out[0];
      }
    }

    std::vector<Step> v;
    std::string fused;
    if (bias_t >= 0)
      fused += "+bias";
    if (act)
      fused += "+act";
    if (res_t >= 0)
      fused += "+residual";
    if (int8 && flat) {
      const Op &da = g_.ops[dq_a], &dw = g_.ops[dq_w];
      const LTensor &qa = T(da.in[0]), &qw = T(dw.in[0]);
      const float sA = da.attrs.at("scales").fa[0];
      const auto &sw = dw.attrs.at("scales").fa;
      int32_t zpA = 0;
      if (da.attrs.count("zps") && !da.attrs.at("zps").ia.empty())
        zpA = (int32_t)da.attrs.at("zps").ia[0];
      // weights stored [N,K] (transpose_b, the layout of torch.nn.Linear): the 8-bit tile kernels read [K,N], so a
      // transposed copy is made -- once per executable when the weights are a constant, the reference's pre-packing
      // of constant weights (docs/CPU_pipeline_overview.md:58); measured on the 4-wave kernel, reading [N,K] tiles
      // in place is no faster than [K,N]
      int64_t K = tb ? qw.shape[1] : qw.shape[0], N = tb ? qw.shape[0] : qw.shape[1], M = qa.numel() / K;
      int w_slot = slot_for(dw.in[0]);
      if (tb) {
        Step cp;
        cp.kind = Step::Elt, cp.op = gcmi::ELT_COPY, cp.once = qw.constant;
        cp.note = qw.constant ? "transpose copy of W [N,K] -> [K,N], once: W is constant" : "transpose copy of W [N,K] -> [K,N]";
        cp.a = w_slot, cp.out = new_slot((size_t)K * N);
        cp.a_dt = cp.out_dt = GCMI_S8, cp.dims = {K, N}, cp.sa = {1, K};
        v.push_back(cp);
        w_slot = cp.out;
      }
      // output_scales = data_scales (x) weight_scales
      // (legacy/core/src/compiler/ir/graph/transform/quantization/graph_reschedule.cpp:220-235)
      std::vector<float> sc((size_t)N);
      for (int64_t nI = 0; nI < N; nI++)
        sc[(size_t)nI] = sA * (sw.size() == 1 ? sw[0] : sw[(size_t)nI]);
      int sc_slot = const_slot(sc.data(), sc.size() * 4);
      int cs_slot = new_slot((size_t)N * 4);
      Step cs;
      cs.kind = Step::ColSum, cs.note = qw.constant ? "colsum(W), once: W is constant" : "colsum(W)";
      cs.a = w_slot, cs.out = cs_slot, cs.K = K, cs.N = N, cs.lda = N;
      cs.op = qw.constant ? 1 : 0;
      v.push_back(cs);
      Step s;
      s.kind = Step::GemmInt8;
      s.note = "Dequantize x2 + MatMul" + fused + (T(cur).dt == DT::bf16 ? "+cast" : "") + " fused";
      s.a = slot_for(da.in[0]), s.b = w_slot, s.out = slot_for(cur);
      s.M = M, s.N = N, s.K = K, s.lda = K, s.ldb = N, s.ldc = N;
      s.a_dt = dt_dnnl(qa.dt), s.zp = zpA, s.aux = cs_slot, s.scales_slot = sc_slot;
      s.bias = bias_t >= 0 ? slot_for((size_t)bias_t) : -1;
      s.act = act, s.out_dt = dt_dnnl(T(cur).dt);
      s.mm_cfg = matmul_config_attrs(mm);
      v.push_back(s);
      skip[dq_a] = skip[dq_w] = claimed[dq_a] = claimed[dq_w] = true;
    } else {
      // plain GEMM, possibly batched
      if (A.dt == DT::f16)
        throw std::logic_error("f16 MatMul is not supported (bf16 and f32 are)");
      // stored 2-D views: 1-D operands become [1,K] / [K,1]
      std::vector<int64_t> as = A.shape, bs = B.shape;
      bool a1 = ra == 1, b1 = rb == 1;
      if (a1)
        as = {1, A.shape[0]};
      if (b1)
        bs = {B.shape[0], 1};
      bool tA = a1 ? false : ta, tB = b1 ? false : tb;
      size_t Ra = as.size(), Rb = bs.size();
      int64_t M = tA ? as[Ra - 1] : as[Ra - 2], K = tA ? as[Ra - 2] : as[Ra - 1];
      int64_t N = tB ? bs[Rb - 2] : bs[Rb - 1];
      int sa_slot = slot_for(mm.in[0]), sb_slot = slot_for(mm.in[1]);
      DT out_dt = T(mm.out[0]).dt;
      if (A.dt == DT::bf16 && tA) {
        // the bf16 kernel reads A row-major [M,K] (B may be stored either way): materialise a transposed A
        // (once per executable when the operand is a constant: the analogue of the reference's weight
        // pre-packing of constant tensors, docs/CPU_pipeline_overview.md:58)
        auto transposed = [&](int slot, std::vector<int64_t> &shp, bool constant) {
          std::vector<int64_t> st = dense_strides(shp), d = shp;
          std::swap(d[d.size() - 1], d[d.size() - 2]);
          std::swap(st[st.size() - 1], st[st.size() - 2]);
          int t = new_slot((size_t)prod(shp, 0, shp.size()) * 2);
          if (d.size() > (size_t)gcmi::ELT_MAX_RANK)
            throw std::logic_error("tensor rank above 6 is not supported");
          Step cp;
          cp.kind = Step::Elt, cp.note = constant ? "transpose copy, once: the operand is constant" : "transpose copy";
          cp.once = constant, cp.op = gcmi::ELT_COPY, cp.a = slot, cp.out = t;
          cp.a_dt = cp.out_dt = GCMI_BF16, cp.dims = d, cp.sa = st;
          v.push_back(cp);
          shp = d;
          return t;
        };
        sa_slot = transposed(sa_slot, as, A.constant), tA = false;
      }
      std::vector<int64_t> ba(as.begin(), as.end() - 2), bb(bs.begin(), bs.end() - 2), bo;
      broadcast_shape(ba, bb, bo);
      int64_t nb = prod(bo, 0, bo.size());
      bool flatten = bb.empty() && !tA; // [..,M,K] x [K,N]: one GEMM over all rows
      int64_t a_mat = as[Ra - 1] * as[Ra - 2], b_mat = bs[Rb - 1] * bs[Rb - 2];
      auto batch_off = [&](const std::vector<int64_t> &bd, int64_t idx) {
        // index into a (possibly broadcast) batch shape aligned to the right of bo
        int64_t off = 0, mul = 1;
        for (int d = (int)bo.size() - 1; d >= 0; d--) {
          int64_t c = idx % bo[d];
          idx /= bo[d];
          int dd = d - ((int)bo.size() - (int)bd.size());
          if (dd >= 0) {
            if (bd[dd] != 1)
              off += c * mul;
            mul *= bd[dd];
          }
        }
        return off;
      };
      int out_slot = slot_for(chain.empty() ? mm.out[0] : cur);
      // batches that advance every operand by a fixed stride (or share it) are one launch; other broadcast
      // patterns fall back to one launch per batch
      auto uniform = [&](const std::vector<int64_t> &bd) { return bd == bo || prod(bd, 0, bd.size()) == 1; };
      const bool strided = !flatten && nb > 1 && nb <= 65535 && uniform(ba) && uniform(bb);
      int64_t reps = flatten || strided ? 1 : nb;
      for (int64_t bi = 0; bi < reps; bi++) {
        Step s;
        s.kind = A.dt == DT::f32 ? Step::GemmF32 : Step::GemmBf16;
        s.note = std::string("MatMul") + fused + (strided ? " (" + std::to_string(nb) + " batches)" : reps > 1 ? " (batched)" : "");
        if (strided) {
          s.batch = nb;
          s.a_bs = ba == bo ? a_mat : 0, s.b_bs = bb == bo ? b_mat : 0, s.c_bs = M * N;
        }
        s.a = sa_slot, s.b = sb_slot, s.out = out_slot;
        s.mm_cfg = matmul_config_attrs(mm);
        s.M = flatten ? M * nb : M, s.N = N, s.K = K;
        s.lda = as[Ra - 1], s.ldb = bs[Rb - 1], s.ldc = N;
        s.ta = tA, s.tb = tB;
        if (!flatten && !strided) {
          s.a_off = batch_off(ba, bi) * a_mat, s.b_off = batch_off(bb, bi) * b_mat, s.out_off = bi * M * N;
        }
        s.bias = bias_t >= 0 ? slot_for((size_t)bias_t) : -1;
        s.bias_dt = bias_t >= 0 ? dt_dnnl(T((size_t)bias_t).dt) : 0;
        s.c = res_t >= 0 ? slot_for((size_t)res_t) : -1;
        s.b_dt = res_t >= 0 ? dt_dnnl(T((size_t)res_t).dt) : 0;
        s.act = act;
        s.out_dt = dt_dnnl(chain.empty() ? out_dt : T(cur).dt);
        v.push_back(s);
      }
      // a MatMul bias that is not a row vector: separate broadcast add, in place
      if (bias_in_matmul && bias_t < 0) {
        const LTensor &bt = T(mm.in[2]), &ot = T(mm.out[0]);
        Step s;
        s.kind = Step::Elt, s.note = "bias add", s.op = gcmi::ELT_ADD;
        s.a = out_slot, s.b = slot_for(mm.in[2]), s.out = out_slot;
        s.a_dt = s.out_dt = dt_dnnl(ot.dt), s.b_dt = dt_dnnl(bt.dt);
        s.dims = ot.shape, s.sa = dense_strides(ot.shape);
        std::vector<int64_t> bst = dense_strides(bt.shape), full(ot.shape.size(), 0);
        for (size_t d = 0; d < bt.shape.size(); d++) {
          size_t od = ot.shape.size() - bt.shape.size() + d;
          full[od] = bt.shape[d] == 1 ? 0 : bst[d];
        }
        s.sb = full;
        if (s.dims.size() > (size_t)gcmi::ELT_MAX_RANK)
          throw std::logic_error("tensor rank above 6 is not supported");
        v.push_back(s);
      }
    }
    for (auto ci : chain)
      skip[ci] = claimed[ci] = true;
    skip[i] = claimed[i] = true;
    skip[last] = false;
    emit_at[last] = v;
  }

  // GCMI_NO_POINTWISE_FUSION=1: one launch per op, for comparing the two ways of running a graph
  // (sums still go to the row-sum kernel, alone)
  const char *no_fuse = getenv("GCMI_NO_POINTWISE_FUSION");
  plan_fusion(skip, claimed, emit_at, !(no_fuse && no_fuse[0] == '1'));

  // ---- emission pass, in op order
  for (size_t i = 0; i < n; i++) {
    if (skip[i])
      continue;
    auto it = emit_at.find(i);
    if (it != emit_at.end()) {
      for (auto &s : it->second)
        steps_.push_back(s);
      continue;
    }
    plan_generic(g_.ops[i]);
  }
}

// ---------------------------------------------------------------------------
// Point-wise fusion: chains and DAGs of element-wise ops of one shape become one launch (a small register program,
// gcmi::FusedParams), and such a group in front of a ReduceSum/ReduceMean is evaluated inside the reduction.  This
// is the part of the reference's producer/consumer fusion (lib/gc/Transforms/IterativeTilingAndFusion.cpp:585-611,
// 652-741) that is not already a GEMM epilogue.  A value leaves the chip only when something other than a
// same-shaped point-wise op or a reduction reads it (a MatMul, a reshape, the caller); values with several
// point-wise readers are recomputed in each group rather than stored.
namespace {
int pointwise_code(const Op &op) {
  const std::string &k = op.kind;
  if (k == "Add")
    return gcmi::ELT_ADD;
  if (k == "Subtract")
    return gcmi::ELT_SUB;
  if (k == "Multiply")
    return gcmi::ELT_MUL;
  if (k == "Divide")
    return gcmi::ELT_DIV;
  if (k == "Maximum")
    return gcmi::ELT_MAX;
  if (k == "ReLU")
    return gcmi::ELT_RELU;
  if (k == "Sigmoid")
    return gcmi::ELT_SIGMOID;
  if (k == "GELU")
    return act_of(op) == GCMI_ACT_GELU_TANH ? gcmi::ELT_GELU_TANH : gcmi::ELT_GELU_ERF;
  if (k == "Pow")
    return gcmi::ELT_POW;
  if (k == "Typecast" || k == "TypeCast")
    return gcmi::ELT_COPY;
  if (k == "Exp")
    return gcmi::ELT_EXP;
  if (k == "Neg")
    return gcmi::ELT_NEG;
  static const std::map<std::string, int> more = {
      {"Minimum", gcmi::ELT_MIN}, {"Abs", gcmi::ELT_ABS},     {"Ceil", gcmi::ELT_CEIL},     {"Floor", gcmi::ELT_FLOOR},
      {"Erf", gcmi::ELT_ERF},     {"Log", gcmi::ELT_LOG},     {"Round", gcmi::ELT_ROUND},   {"Rsqrt", gcmi::ELT_RSQRT},
      {"Sqrt", gcmi::ELT_SQRT},   {"Square", gcmi::ELT_SQUARE}, {"Tanh", gcmi::ELT_TANH},   {"Reciprocal", gcmi::ELT_RECIP}};
  auto it = more.find(k);
  return it == more.end() ? -1 : it->second;
}
bool storage_float(DT d) { return d == DT::f32 || d == DT::bf16 || d == DT::f16; }
} // namespace

static int fused_registers(const Step &s);

std::vector<int64_t> squeezed(const std::vector<int64_t> &shape) {
  std::vector<int64_t> r;
  for (auto d : shape)
    if (d != 1)
      r.push_back(d);
  return r;
}

void Executable::plan_fusion(std::vector<bool> &skip, const std::vector<bool> &claimed,
                             std::map<size_t, std::vector<Step>> &emit_at, bool groups) {
  const size_t n = g_.ops.size();
  auto T = [&](size_t id) -> const LTensor & { return g_.tensors.at(id); };
  // a reshape is a view of its source: readers of the view are readers of the source, and shapes are compared
  // without their unit dims ([1,32,4096] and [32,4096] walk memory alike)
  auto base = [&](size_t t) {
    while (T(t).alias_of >= 0)
      t = (size_t)T(t).alias_of;
    return t;
  };
  auto view_op = [&](size_t i) { return g_.ops[i].kind == "Reshape"; };
  std::map<size_t, std::vector<size_t>> consumers;
  std::map<size_t, size_t> producer;
  for (size_t i = 0; i < n; i++) {
    if (view_op(i))
      continue;
    for (auto id : g_.ops[i].in)
      consumers[base(id)].push_back(i);
    for (auto id : g_.ops[i].out)
      producer[id] = i;
  }
  std::set<size_t> outs;
  for (auto id : g_.output_ids)
    outs.insert(base(id));

  // ops no GEMM or attention group has taken (as the matching pass left them: this pass must not see its own marks)
  std::vector<bool> is_free(n);
  for (size_t i = 0; i < n; i++)
    is_free[i] = !skip[i] && !claimed[i] && !emit_at.count(i);
  auto fusable = [&](size_t i) {
    const Op &o = g_.ops[i];
    if (!groups || !is_free[i] || pointwise_code(o) < 0 || o.out.size() != 1)
      return false;
    const LTensor &ot = T(o.out[0]);
    if (!storage_float(ot.dt) || ot.shape.size() > (size_t)gcmi::ELT_MAX_RANK || !is_dense(ot))
      return false;
    for (auto id : o.in)
      if (!storage_float(T(id).dt) || !is_dense(T(id)))
        return false;
    return true;
  };
  auto reduction = [&](size_t i) {
    const Op &o = g_.ops[i];
    if (!is_free[i] || !(o.kind == "ReduceSum" || o.kind == "ReduceMean"))
      return false;
    if (!o.attrs.count("axes") || o.attrs.at("axes").ia.empty())
      return false; // nothing is reduced: a copy (plan_generic)
    const LTensor &it = T(o.in[0]);
    return storage_float(it.dt) && storage_float(T(o.out[0]).dt) && it.shape.size() <= (size_t)gcmi::ELT_MAX_RANK &&
           is_dense(it);
  };
  std::set<size_t> forced; // tensors a group could not take in (size limits): they are stored after all
  // does anything read this tensor from memory?
  auto stored = [&](size_t t) {
    if (outs.count(t) || forced.count(t))
      return true;
    auto it = consumers.find(t);
    if (it == consumers.end() || it->second.empty())
      return true;
    for (size_t c : it->second) {
      if (fusable(c) && squeezed(T(g_.ops[c].out[0]).shape) == squeezed(T(t).shape))
        continue;
      if (reduction(c))
        continue;
      return true;
    }
    return false;
  };

  std::set<size_t> taken_reductions;
  std::vector<size_t> fused_roots;
  for (size_t i = n; i-- > 0;) {
    const Op &root = g_.ops[i];
    const bool red_root = reduction(i);
    if (red_root && taken_reductions.count(i))
      continue;
    if (!red_root && !(fusable(i) && stored(base(root.out[0]))))
      continue;
    // the group: point-wise ops on the row shape (`post`; without a sum this is the whole group), optionally a
    // sum, and point-wise ops on the full shape in front of the sum (`pre`)
    std::set<size_t> post, pre;
    long red = red_root ? (long)i : -1;
    std::vector<int64_t> row_dims = squeezed(T(root.out[0]).shape), full_dims;
    if (red_root)
      full_dims = squeezed(T(root.in[0]).shape);
    // tensors (canonical) currently read from memory, per phase
    std::vector<std::pair<size_t, int>> inputs; // phase 0 = pre, 1 = post
    auto add_input = [&](std::vector<std::pair<size_t, int>> &v, size_t t, int phase) {
      std::pair<size_t, int> e(base(t), phase);
      if (std::find(v.begin(), v.end(), e) == v.end())
        v.push_back(e);
    };
    if (red_root) {
      add_input(inputs, root.in[0], 0);
    } else {
      post.insert(i);
      for (auto id : root.in)
        add_input(inputs, id, 1);
    }
    auto inside = [&](size_t t, int phase) {
      auto pit = producer.find(t);
      if (pit == producer.end())
        return false;
      if (phase == 1 && red >= 0 && (long)pit->second == red)
        return true;
      return (phase == 1 ? post : pre).count(pit->second) > 0;
    };
    std::set<std::pair<size_t, int>> declined;
    for (bool grew = true; grew;) {
      grew = false;
      for (size_t k = 0; k < inputs.size(); k++) {
        const size_t t = inputs[k].first;
        const int phase = inputs[k].second;
        auto pit = producer.find(t);
        if (declined.count(inputs[k]) || pit == producer.end() || T(t).has_splat || stored(t))
          continue;
        const size_t po = pit->second;
        const bool take_sum = phase == 1 && red < 0 && reduction(po) && consumers[t].size() == 1 &&
                              squeezed(T(t).shape) == row_dims;
        const bool take_op = fusable(po) && squeezed(T(t).shape) == (phase == 1 ? row_dims : full_dims);
        if (!take_sum && !take_op)
          continue;
        std::vector<std::pair<size_t, int>> next;
        for (auto &x : inputs)
          if (x != inputs[k])
            next.push_back(x);
        const int in_phase = take_sum ? 0 : phase;
        for (auto x : g_.ops[po].in)
          if (!inside(base(x), in_phase))
            add_input(next, x, in_phase);
        const size_t count = post.size() + pre.size() + (red >= 0 || take_sum ? 1 : 0) + (take_sum ? 0 : 1);
        // two inputs of slack: one tensor read through different broadcasts counts once here and twice below
        if (count > (size_t)gcmi::FUSED_MAX_INS || next.size() + 2 > (size_t)gcmi::FUSED_MAX_IN) {
          declined.insert(inputs[k]);
          forced.insert(t);
          continue;
        }
        if (take_sum) {
          red = (long)po;
          full_dims = squeezed(T(g_.ops[po].in[0]).shape);
        } else {
          (phase == 1 ? post : pre).insert(po);
        }
        inputs = next;
        grew = true;
        break;
      }
    }
    if (red < 0 && post.size() == 1 && !groups)
      continue; // one launch per op was asked for: the plain element-wise kernel
    // (otherwise a lone op is a group of one: four elements per thread, vector moves, a generated kernel)

    // ---- iteration space: [kept dims..., reduced dims...] of the sum's input, or the point-wise shape
    Step s;
    s.kind = Step::Fused;
    std::vector<int> place; // position among the non-unit dims of the full shape -> iteration dim
    size_t n_kept = row_dims.size();
    if (red >= 0) {
      const Op &ro = g_.ops[(size_t)red];
      const std::vector<int64_t> &fs = T(ro.in[0]).shape;
      std::vector<int64_t> axes;
      if (ro.attrs.count("axes"))
        axes = ro.attrs.at("axes").ia;
      auto ca = canonical_axes(axes, (int64_t)fs.size());
      std::vector<int64_t> kept, reduced;
      std::vector<bool> is_red;
      for (size_t d = 0; d < fs.size(); d++) {
        if (fs[d] == 1)
          continue;
        bool r = std::find(ca.begin(), ca.end(), (int64_t)d) != ca.end();
        (r ? reduced : kept).push_back(fs[d]);
        is_red.push_back(r);
      }
      n_kept = kept.size();
      place.resize(is_red.size());
      int nk = 0, nr = 0;
      for (size_t q = 0; q < is_red.size(); q++)
        place[q] = is_red[q] ? (int)n_kept + nr++ : nk++;
      s.dims = kept;
      s.dims.insert(s.dims.end(), reduced.begin(), reduced.end());
      s.n_red = 1;
      for (auto d : reduced)
        s.n_red *= d;
      s.mean = ro.kind == "ReduceMean";
      if (kept != squeezed(T(ro.out[0]).shape))
        throw std::logic_error("reduction whose result shape does not match its kept dims");
    } else {
      s.dims = row_dims;
    }
    if (s.dims.size() > (size_t)gcmi::ELT_MAX_RANK)
      throw std::logic_error("tensor rank above 6 is not supported");

    // strides of operand x, as the member whose result has shape `ms` reads it, over the iteration dims
    auto strides_of = [&](size_t x, const std::vector<int64_t> &ms, int phase) {
      const LTensor &t = T(x);
      std::vector<int64_t> st = dense_strides(t.shape), full(ms.size(), 0), it(s.dims.size(), 0);
      if (!t.has_splat)
        for (size_t d = 0; d < t.shape.size(); d++)
          full[ms.size() - t.shape.size() + d] = t.shape[d] == 1 ? 0 : st[d];
      size_t q = 0;
      for (size_t d = 0; d < ms.size(); d++) {
        if (ms[d] == 1)
          continue;
        const size_t pos = (phase == 0 && red >= 0) ? (size_t)place[q] : q; // post-phase dims are the leading (kept) ones
        it[pos] = full[d];
        q++;
      }
      return it;
    };
    struct In {
      size_t tensor; // as named by the reader (a view keeps its own shape)
      int phase;
      std::vector<int64_t> str;
    };
    std::vector<In> ins_pre, ins_post;
    std::map<size_t, int> reg_of_op;   // member op (or the sum) -> register, filled as instructions are numbered
    std::vector<size_t> order_pre(pre.begin(), pre.end()), order_post(post.begin(), post.end());
    // pass 1: collect inputs
    auto operand_input = [&](size_t x, const std::vector<int64_t> &ms, int phase) -> int {
      std::vector<In> &v = phase == 0 ? ins_pre : ins_post;
      std::vector<int64_t> st = strides_of(x, ms, phase);
      for (size_t k = 0; k < v.size(); k++)
        if (base(v[k].tensor) == base(x) && v[k].str == st)
          return (int)k;
      v.push_back({x, phase, st});
      return (int)v.size() - 1;
    };
    struct Use {
      bool is_input;
      int index;    // input index within its phase, or producing op
      size_t op;
    };
    auto classify = [&](size_t x, const std::vector<int64_t> &ms, int phase) {
      Use u{};
      const size_t b = base(x);
      if (inside(b, phase)) {
        u.is_input = false;
        u.op = producer.at(b);
      } else {
        u.is_input = true;
        u.index = operand_input(x, ms, phase);
      }
      return u;
    };
    std::vector<std::vector<Use>> uses_pre, uses_post;
    for (size_t m : order_pre) {
      std::vector<Use> u;
      for (auto x : g_.ops[m].in)
        u.push_back(classify(x, T(g_.ops[m].out[0]).shape, 0));
      uses_pre.push_back(u);
    }
    Use sum_use{};
    if (red >= 0)
      sum_use = classify(g_.ops[(size_t)red].in[0], T(g_.ops[(size_t)red].in[0]).shape, 0);
    for (size_t m : order_post) {
      std::vector<Use> u;
      for (auto x : g_.ops[m].in)
        u.push_back(classify(x, T(g_.ops[m].out[0]).shape, 1));
      uses_post.push_back(u);
    }
    const int n_in_pre = (int)ins_pre.size(), n_in = n_in_pre + (int)ins_post.size();
    if (n_in > gcmi::FUSED_MAX_IN || n_in < 1)
      throw std::logic_error("point-wise fusion: input count out of range");
    for (auto &v : {ins_pre, ins_post})
      for (auto &e : v) {
        s.f_in.push_back(slot_for(e.tensor));
        s.f_in_dt.push_back(dt_dnnl(T(e.tensor).dt));
        s.f_str.push_back(e.str);
        s.f_in_tensor.push_back(base(e.tensor));
      }
    auto reg_of = [&](const Use &u, int phase) {
      return u.is_input ? (phase == 0 ? u.index : n_in_pre + u.index) : reg_of_op.at(u.op);
    };
    std::string names_pre, names_post;
    auto emit_member = [&](size_t m, const std::vector<Use> &u, int phase, std::string &names) {
      const Op &o = g_.ops[m];
      Step::FIns f;
      f.op = pointwise_code(o);
      f.a = reg_of(u[0], phase);
      f.b = u.size() > 1 ? reg_of(u[1], phase) : f.a;
      f.dt = dt_dnnl(T(o.out[0]).dt);
      f.imm = o.kind == "Pow" ? o.attr_f32("beta", 1.0f) : 0.0f;
      reg_of_op[m] = n_in + (int)s.f_ins.size();
      s.f_ins.push_back(f);
      names += (names.empty() ? "" : "+") + o.kind;
    };
    for (size_t q = 0; q < order_pre.size(); q++)
      emit_member(order_pre[q], uses_pre[q], 0, names_pre);
    s.sum_ins = -1;
    if (red >= 0) {
      Step::FIns f;
      f.op = gcmi::ELT_ROWSUM;
      f.a = f.b = reg_of(sum_use, 0);
      f.dt = dt_dnnl(T(g_.ops[(size_t)red].out[0]).dt);
      f.imm = 0.0f;
      s.sum_ins = (int)s.f_ins.size();
      reg_of_op[(size_t)red] = n_in + s.sum_ins;
      s.f_ins.push_back(f);
    }
    for (size_t q = 0; q < order_post.size(); q++)
      emit_member(order_post[q], uses_post[q], 1, names_post);
    s.n_in_pre = n_in_pre;
    s.out = slot_for(root.out[0]);
    s.out_dt = dt_dnnl(T(root.out[0]).dt);
    s.red_reg = reg_of_op.at(i);
    if (red >= 0) {
      const std::string rk = g_.ops[(size_t)red].kind;
      s.note = (names_post.empty() ? "" : names_post + " of ") + rk + (names_pre.empty() ? "" : " of " + names_pre);
      taken_reductions.insert((size_t)red);
      skip[(size_t)red] = true;
    } else {
      s.note = names_post;
    }
    for (size_t m : pre)
      skip[m] = true, s.f_members.push_back(m);
    for (size_t m : post)
      skip[m] = true, s.f_members.push_back(m);
    if (red >= 0)
      s.f_members.push_back((size_t)red);
    s.f_out_tensor = base(root.out[0]);
    s.f_place = place;
    if (fused_registers(s) > gcmi::FUSED_MAX_PHYS)
      throw std::logic_error("point-wise group with more than " + std::to_string(gcmi::FUSED_MAX_PHYS) +
                             " values alive at once (" + s.note + ")");
    skip[i] = false;
    emit_at[i] = {s};
    fused_roots.push_back(i);
  }

  // ---- a row statistic and the point-wise group that scales by it become one launch (a normalisation): the
  // second group runs as a second pass over the row inside the row kernel
  std::sort(fused_roots.begin(), fused_roots.end());
  for (size_t i2 : fused_roots) {
    auto it2 = emit_at.find(i2);
    if (it2 == emit_at.end() || it2->second.size() != 1)
      continue;
    Step &s2 = it2->second[0];
    if (s2.kind != Step::Fused || s2.sum_ins >= 0)
      continue;
    for (size_t k = 0; k < s2.f_in_tensor.size(); k++) {
      const size_t r = s2.f_in_tensor[k];
      auto pit = producer.find(r);
      if (pit == producer.end() || outs.count(r))
        continue;
      // the group that writes r: emitted at its last op
      size_t i1 = n;
      for (size_t cand : fused_roots)
        if (cand < i2 && emit_at.count(cand) && emit_at[cand].size() == 1 && emit_at[cand][0].kind == Step::Fused &&
            emit_at[cand][0].sum_ins >= 0 && emit_at[cand][0].row_end < 0 && emit_at[cand][0].f_out_tensor == r)
          i1 = cand;
      if (i1 == n)
        continue;
      const Step &s1 = emit_at[i1][0];
      // nothing but this group reads r, and it reads it one way (one input)
      if (std::count(s2.f_in_tensor.begin(), s2.f_in_tensor.end(), r) != 1)
        continue;
      bool only_here = true;
      for (size_t c : consumers[r])
        only_here = only_here && std::find(s2.f_members.begin(), s2.f_members.end(), c) != s2.f_members.end();
      // an op with several point-wise readers is a member of each reader's group (it is recomputed there): no other
      // group may load r either (a layer normalisation reads the mean in the variance group and in the scaling)
      for (auto &other : emit_at)
        for (const Step &so : other.second)
          if (other.first != i2 && so.kind == Step::Fused &&
              std::find(so.f_in_tensor.begin(), so.f_in_tensor.end(), r) != so.f_in_tensor.end())
            only_here = false;
      // the same non-unit dims, and r broadcast exactly along the summed ones
      const size_t nd = s1.dims.size();
      if (!only_here || s1.f_place.size() != nd || s2.dims.size() != nd)
        continue;
      bool same = true;
      for (size_t q = 0; q < nd; q++)
        same = same && s2.dims[q] == s1.dims[(size_t)s1.f_place[q]];
      const size_t n_kept = nd - [&] {
        size_t c = 0;
        int64_t in_row = 1;
        for (size_t d = nd; d-- > 0 && in_row < s1.n_red;)
          in_row *= s1.dims[d], c++;
        return c;
      }();
      std::vector<int64_t> kept(s1.dims.begin(), s1.dims.begin() + (long)n_kept), kst = dense_strides(kept);
      for (size_t q = 0; q < nd && same; q++) {
        const size_t pos = (size_t)s1.f_place[q];
        same = s2.f_str[k][q] == (pos < n_kept ? kst[pos] : 0);
      }
      const size_t n_in_new = s1.f_in.size() + s2.f_in.size() - 1, n_ins_new = s1.f_ins.size() + s2.f_ins.size();
      if (!same || n_in_new > (size_t)gcmi::FUSED_MAX_IN || n_ins_new > (size_t)gcmi::FUSED_MAX_INS)
        continue;
      // one workgroup walks a row twice: worth it when there are rows enough to fill the GPU; a few long rows
      // (32 tokens x 4096) are quicker as a row kernel and a point-wise kernel spread over all compute units
      int64_t rows = 1;
      for (size_t d = 0; d < n_kept; d++)
        rows *= s1.dims[d];
      // (that holds for the library's generic row kernel, whose fixed cost per workgroup is high; a generated
      // kernel is quicker as one launch at every row count)
      const char *min_rows = getenv("GCMI_ROW_MERGE_MIN_ROWS"), *no_gen = getenv("GCMI_NO_GENERATED_KERNELS"); // tuning knob
      if (rows < (min_rows ? atoll(min_rows) : no_gen && no_gen[0] == '1' ? 512 : 1))
        continue;
      Step m = s1;
      m.note = s2.note + " after " + s1.note;
      m.n_in_row = (int)s1.f_in.size();
      m.row_end = (int)s1.f_ins.size();
      const int shift1 = (int)n_in_new - (int)s1.f_in.size(); // results of the first group move up by this much
      for (auto &f : m.f_ins) {
        if (f.a >= (int)s1.f_in.size())
          f.a += shift1;
        if (f.b >= (int)s1.f_in.size())
          f.b += shift1;
      }
      const int r_reg = s1.red_reg + shift1;
      auto permute = [&](const std::vector<int64_t> &by_dim) {
        std::vector<int64_t> it(nd, 0);
        for (size_t q = 0; q < nd; q++)
          it[(size_t)s1.f_place[q]] = by_dim[q];
        return it;
      };
      std::vector<int> in_map(s2.f_in.size(), -1);
      for (size_t x = 0; x < s2.f_in.size(); x++) {
        if (x == k)
          continue;
        in_map[x] = (int)m.f_in.size();
        m.f_in.push_back(s2.f_in[x]);
        m.f_in_dt.push_back(s2.f_in_dt[x]);
        m.f_str.push_back(permute(s2.f_str[x]));
        m.f_in_tensor.push_back(s2.f_in_tensor[x]);
      }
      auto map2 = [&](int reg) {
        if (reg == (int)k)
          return r_reg;
        if (reg < (int)s2.f_in.size())
          return in_map[(size_t)reg];
        return (int)n_in_new + (int)s1.f_ins.size() + (reg - (int)s2.f_in.size());
      };
      for (auto f : s2.f_ins) {
        f.a = map2(f.a), f.b = map2(f.b);
        m.f_ins.push_back(f);
      }
      m.out = s2.out, m.out_dt = s2.out_dt, m.red_reg = map2(s2.red_reg);
      m.out_str = permute(dense_strides(s2.dims));
      m.f_members.insert(m.f_members.end(), s2.f_members.begin(), s2.f_members.end());
      m.f_out_tensor = s2.f_out_tensor;
      if (fused_registers(m) > gcmi::FUSED_MAX_PHYS)
        continue;
      skip[i1] = true;
      emit_at.erase(i1);
      it2->second[0] = m;
      break;
    }
  }
}

// ---------------------------------------------------------------------------
void Executable::plan_generic(const Op &op) {
  auto T = [&](size_t id) -> const LTensor & { return g_.tensors.at(id); };
  const std::string &k = op.kind;
  const LTensor &out = T(op.out[0]);
  if (out.shape.size() > (size_t)gcmi::ELT_MAX_RANK)
    throw std::logic_error("tensor rank above 6 is not supported");
  auto bstrides = [&](const LTensor &t) {
    std::vector<int64_t> st = dense_strides(t.shape), full(out.shape.size(), 0);
    if (t.has_splat)
      return full;
    for (size_t d = 0; d < t.shape.size(); d++) {
      size_t od = out.shape.size() - t.shape.size() + d;
      full[od] = t.shape[d] == 1 ? 0 : st[d];
    }
    return full;
  };
  Step s;
  s.kind = Step::Elt;
  s.note = k;
  if (k == "Reshape") {
    (void)slot_for(op.out[0]); // a view: no work
    return;
  }
  if (k == "Transpose" || k == "BroadcastTo") {
    const LTensor &in = T(op.in[0]);
    std::vector<int64_t> ist = dense_strides(in.shape), st(out.shape.size(), 0);
    if (k == "Transpose") {
      const auto &perm = op.attrs.at("perm").ia;
      for (size_t d = 0; d < perm.size(); d++)
        st[d] = ist[(size_t)perm[d]];
    } else {
      const auto &added = op.attrs.at("dims").ia;
      size_t src = 0;
      for (size_t d = 0; d < out.shape.size(); d++)
        if (std::find(added.begin(), added.end(), (int64_t)d) == added.end())
          st[d] = in.has_splat ? 0 : ist[src++];
    }
    s.note = k == "Transpose" ? "Transpose (strided copy)" : "BroadcastTo (stride-0 copy)";
    s.op = gcmi::ELT_COPY;
    s.a = slot_for(op.in[0]), s.out = slot_for(op.out[0]);
    s.a_dt = dt_dnnl(in.dt), s.out_dt = dt_dnnl(out.dt);
    s.dims = out.shape, s.sa = st;
    steps_.push_back(std::move(s));
    return;
  }
  if (pointwise_code(op) >= 0 && op.in.size() == 2) {
    s.op = pointwise_code(op);
    s.a = slot_for(op.in[0]), s.b = slot_for(op.in[1]), s.out = slot_for(op.out[0]);
    s.a_dt = dt_dnnl(T(op.in[0]).dt), s.b_dt = dt_dnnl(T(op.in[1]).dt), s.out_dt = dt_dnnl(out.dt);
    s.dims = out.shape, s.sa = bstrides(T(op.in[0])), s.sb = bstrides(T(op.in[1]));
  } else if (pointwise_code(op) >= 0 && op.in.size() == 1) {
    s.op = pointwise_code(op);
    s.alpha = k == "Pow" ? op.attr_f32("beta", 1.0f) : 0.0f;
    s.a = slot_for(op.in[0]), s.out = slot_for(op.out[0]);
    s.a_dt = dt_dnnl(T(op.in[0]).dt), s.out_dt = dt_dnnl(out.dt);
    s.dims = {out.numel()}, s.sa = {1};
  } else if (k == "Dequantize" || k == "Quantize") {
    const LTensor &in = T(op.in[0]);
    s.op = k == "Dequantize" ? gcmi::ELT_DEQUANT : gcmi::ELT_QUANT;
    s.a = slot_for(op.in[0]), s.out = slot_for(op.out[0]);
    s.a_dt = dt_dnnl(in.dt), s.out_dt = dt_dnnl(out.dt);
    s.dims = out.shape, s.sa = dense_strides(out.shape);
    const auto &sc = op.attrs.at("scales").fa;
    s.n_scales = (int)sc.size();
    s.scales_slot = const_slot(sc.data(), sc.size() * 4);
    std::vector<int32_t> zp(sc.size(), 0);
    if (op.attrs.count("zps")) {
      const auto &z = op.attrs.at("zps").ia;
      for (size_t i = 0; i < zp.size() && !z.empty(); i++)
        zp[i] = (int32_t)(z.size() == 1 ? z[0] : z[i]);
    }
    s.zps_slot = const_slot(zp.data(), zp.size() * 4);
    int64_t ax = op.attr_s64("axis", 1);
    if (ax < 0)
      ax += (int64_t)out.shape.size();
    s.ch_axis = (int)ax;
  } else if ((k == "ReduceSum" || k == "ReduceMean") && (!op.attrs.count("axes") || op.attrs.at("axes").ia.empty())) {
    // no axes: the op returns its operand
    s.note = k + " without axes (copy)";
    s.op = gcmi::ELT_COPY;
    s.a = slot_for(op.in[0]), s.out = slot_for(op.out[0]);
    s.a_dt = dt_dnnl(T(op.in[0]).dt), s.out_dt = dt_dnnl(out.dt);
    s.dims = {out.numel()}, s.sa = {1};
  } else if (k == "ReduceSum" || k == "ReduceMean") {
    const LTensor &in = T(op.in[0]);
    std::vector<int64_t> axes;
    if (op.attrs.count("axes"))
      axes = op.attrs.at("axes").ia;
    auto ca = canonical_axes(axes, (int64_t)in.shape.size());
    auto st = dense_strides(in.shape);
    s.kind = Step::Reduce;
    s.a = slot_for(op.in[0]), s.out = slot_for(op.out[0]);
    s.a_dt = dt_dnnl(in.dt);
    s.mean = k == "ReduceMean";
    for (size_t d = 0; d < in.shape.size(); d++) {
      bool red = std::find(ca.begin(), ca.end(), (int64_t)d) != ca.end();
      (red ? s.rdims : s.kdims).push_back(in.shape[d]);
      (red ? s.rstr : s.kstr).push_back(st[d]);
    }
  } else if (k == "SoftMax") {
    const LTensor &in = T(op.in[0]);
    int64_t r = (int64_t)in.shape.size(), ax = op.attr_s64("axis", 1);
    if (ax < 0)
      ax += r;
    s.kind = Step::Softmax;
    s.a = slot_for(op.in[0]), s.out = slot_for(op.out[0]);
    s.a_dt = dt_dnnl(in.dt), s.out_dt = dt_dnnl(out.dt);
    s.outer = prod(in.shape, 0, (size_t)ax), s.len = in.shape[(size_t)ax], s.inner = prod(in.shape, (size_t)ax + 1, (size_t)r);
  } else {
    throw std::logic_error("Unsupported operation: " + k);
  }
  steps_.push_back(std::move(s));
}

// the parameter block of a fused step, without the operand addresses
static void fill_fused_params(const Step &s, gcmi::FusedParams &p) {
  p.n_in = (int)s.f_in.size(), p.n_in_pre = s.n_in_pre, p.n_ins = (int)s.f_ins.size(), p.sum_ins = s.sum_ins;
  const size_t r = s.dims.size(), pad = gcmi::ELT_MAX_RANK - r;
  p.n = 1;
  for (int d = 0; d < gcmi::ELT_MAX_RANK; d++)
    p.dims[d] = 1;
  for (size_t d = 0; d < r; d++)
    p.dims[pad + d] = s.dims[d], p.n *= s.dims[d];
  for (int k = 0; k < p.n_in; k++) {
    p.in_dt[k] = s.f_in_dt[(size_t)k];
    for (size_t d = 0; d < r; d++)
      p.in_str[k][pad + d] = s.f_str[(size_t)k][d];
  }
  for (int j = 0; j < p.n_ins; j++) {
    const Step::FIns &f = s.f_ins[(size_t)j];
    p.ins[j].op = f.op, p.ins[j].a = f.a, p.ins[j].b = f.b, p.ins[j].dt = f.dt, p.ins[j].imm = f.imm;
  }
  p.out_dt = s.out_dt, p.out_reg = s.red_reg;
  p.n_red = s.sum_ins >= 0 ? s.n_red : 1, p.mean = s.mean;
  const bool second_pass = s.row_end >= 0;
  p.n_in_row = second_pass ? s.n_in_row : p.n_in, p.row_end = second_pass ? s.row_end : p.n_ins;
  for (size_t d = 0; d < r && second_pass; d++)
    p.out_str[pad + d] = s.out_str[d];
}

// physical registers the step's program needs (the kernels hold gcmi::FUSED_MAX_PHYS)
static int fused_registers(const Step &s) {
  gcmi::FusedParams p{};
  fill_fused_params(s, p);
  return gcmi::fused_allocate(p);
}

// Kernels specialised for the fused groups of this plan (jit/fused_jit.h).  GCMI_NO_GENERATED_KERNELS=1 keeps the
// library's interpreter kernels, which compute the same bits (tests compare the two).  A group the generator does not
// cover, or a compiler that is missing or fails, also leaves the interpreter in place.
std::vector<gcjit::FusedKernelSource> Executable::generated_kernels() const {
  std::vector<gcjit::FusedKernelSource> ks;
  for (size_t i = 0; i < steps_.size(); i++) {
    const Step &s = steps_[i];
    if (s.kind == Step::Softmax && s.inner == 1) {
      gcjit::FusedKernelSource k;
      if (gcjit::generate_softmax(s.outer, s.len, s.a_dt, s.out_dt, "gcmi_fused_step" + std::to_string(i), k)) {
        k.source = "// SoftMax\n" + k.source;
        ks.push_back(std::move(k));
      }
      continue;
    }
    if (s.kind != Step::Fused)
      continue;
    gcmi::FusedParams p{};
    fill_fused_params(s, p);
    int same_as[gcmi::FUSED_MAX_IN];
    for (int k = 0; k < p.n_in; k++) {
      same_as[k] = -1;
      for (int j = 0; j < k && same_as[k] < 0; j++)
        if (s.f_in[(size_t)j] == s.f_in[(size_t)k] && s.f_str[(size_t)j] == s.f_str[(size_t)k] && p.in_dt[j] == p.in_dt[k])
          same_as[k] = j;
    }
    gcjit::FusedKernelSource k;
    if (gcjit::generate_fused(p, same_as, "gcmi_fused_step" + std::to_string(i), k)) {
      k.source = "// " + s.note + "\n" + k.source;
      ks.push_back(std::move(k));
    }
  }
  return ks;
}

static std::atomic<long> g_generated_launches{0};
long Executable::generated_launches() { return g_generated_launches.load(); }

void Executable::build_generated_kernels() {
  const char *off = getenv("GCMI_NO_GENERATED_KERNELS");
  if (off && off[0] == '1')
    return;
  const std::vector<gcjit::FusedKernelSource> ks = generated_kernels();
  if (ks.empty())
    return;
  std::string error;
  jit_module_ = gcjit::Module::build(ks, error);
  if (!jit_module_) {
    const char *strict = getenv("GCMI_GENERATED_KERNELS_REQUIRED");
    if (strict && strict[0] == '1')
      throw std::runtime_error("generated kernels: " + error);
    return;
  }
  for (const gcjit::FusedKernelSource &k : ks) {
    const size_t i = (size_t)std::stoul(k.name.substr(strlen("gcmi_fused_step")));
    Step &s = steps_[i];
    s.jit_fn = jit_module_->function(k.name);
    s.jit_grid = k.grid, s.jit_block = k.block, s.jit_vectors = k.quad;
  }
}

// ---------------------------------------------------------------------------
void Executable::launch(const Step &s) {
  auto P = [&](int slot) -> char * { return slot < 0 ? nullptr : (char *)ptr_[(size_t)slot]; };
  switch (s.kind) {
  case Step::GemmF32:
    gc_check(gcmi_gemm_f32_batched((const float *)P(s.a) + s.a_off, (const float *)P(s.b) + s.b_off,
                                   (float *)P(s.out) + s.out_off, s.batch, s.M, s.N, s.K, s.lda, s.ldb, s.ldc, s.a_bs, s.b_bs,
                                   s.c_bs, s.ta, s.tb, (const float *)P(s.bias), s.act, stream_),
             "MatMul f32");
    break;
  case Step::GemmBf16:
    // s.c: the residual tensor (same shape as the result), s.b_dt its type
    gc_check(gcmi_gemm_bf16_ws(P(s.a) + s.a_off * 2, P(s.b) + s.b_off * 2,
                               P(s.out) + s.out_off * (s.out_dt == GCMI_BF16 ? 2 : 4), s.batch, s.M, s.N, s.K, s.lda, s.ldb,
                               s.ldc, s.a_bs, s.b_bs, s.c_bs, s.tb ? 1 : 0, P(s.bias), s.bias_dt ? s.bias_dt : GCMI_BF16,
                               s.act, P(s.c), s.N, s.b_dt ? s.b_dt : GCMI_BF16, s.out_dt, P(s.ws),
                               s.ws >= 0 ? slots_[(size_t)s.ws].bytes : 0, s.mm_cfg.size() == 9 ? s.mm_cfg.data() : nullptr,
                               stream_),
             "MatMul bf16");
    break;
  case Step::ColSum:
    if (s.op == 1 && colsum_valid_[s.out])
      break; // constant weight: already summed
    gc_check(gcmi_colsum_s8(P(s.a), s.K, s.N, s.lda, (int32_t *)P(s.out), stream_), "colsum");
    colsum_valid_[s.out] = true;
    break;
  case Step::GemmInt8:
    gc_check(gcmi_gemm_int8_cfg(P(s.a), s.a_dt, P(s.b), P(s.out), s.M, s.N, s.K, s.lda, s.ldb, s.ldc, (const int32_t *)P(s.aux),
                                s.zp, (const float *)P(s.scales_slot), (const float *)P(s.bias), s.act, s.out_dt,
                                s.mm_cfg.size() == 9 ? s.mm_cfg.data() : nullptr, stream_),
             "MatMul int8");
    break;
  case Step::Mha: {
    float scale = s.scale;
    if (s.scale_slot >= 0) {
      // a one-element input tensor: read it back (blocks until staging is done)
      uint32_t raw = 0;
      hip_check(hipMemcpyAsync(&raw, P(s.scale_slot), s.a_dt == GCMI_BF16 ? 2 : 4, hipMemcpyDeviceToHost, stream_), "read scale");
      hip_check(hipStreamSynchronize(stream_), "read scale");
      float v;
      if (s.a_dt == GCMI_BF16)
        raw <<= 16;
      memcpy(&v, &raw, 4);
      scale = s.scale_div ? 1.0f / v : v;
    }
    gc_check(gcmi_mha_fwd_bf16_ws(P(s.a), P(s.b), P(s.c), (const float *)P(s.mask), s.mask_ld, P(s.out), s.BH, s.Sq, s.Sk,
                                  s.D, scale, GCMI_MHA_SKIP_MASKED | (s.classes_valid ? GCMI_MHA_CLASSES_VALID : 0), P(s.ws),
                                  s.ws >= 0 ? slots_[(size_t)s.ws].bytes : 0, stream_),
             "attention");
    break;
  }
  case Step::MhaClassify:
    gc_check(gcmi_mha_classify_mask((const float *)P(s.a), s.mask_ld, s.Sq, s.Sk, s.D, P(s.out), slots_[(size_t)s.out].bytes,
                                    stream_),
             "mask tile classes");
    break;
  case Step::Elt: {
    gcmi::EltParams p{};
    p.a = P(s.a), p.b = P(s.b), p.out = P(s.out);
    p.op = s.op, p.a_dt = s.a_dt, p.b_dt = s.b_dt, p.out_dt = s.out_dt, p.alpha = s.alpha;
    size_t r = s.dims.size(), pad = gcmi::ELT_MAX_RANK - r;
    p.n = 1;
    for (int d = 0; d < gcmi::ELT_MAX_RANK; d++)
      p.dims[d] = 1, p.sa[d] = 0, p.sb[d] = 0;
    for (size_t d = 0; d < r; d++) {
      p.dims[pad + d] = s.dims[d];
      p.sa[pad + d] = s.sa.empty() ? 0 : s.sa[d];
      p.sb[pad + d] = s.sb.empty() ? 0 : s.sb[d];
      p.n *= s.dims[d];
    }
    p.scales = (const float *)P(s.scales_slot), p.zps = (const int32_t *)P(s.zps_slot);
    p.n_scales = s.n_scales, p.ch_axis = s.ch_axis >= 0 ? (int)pad + s.ch_axis : -1;
    gc_check(gcmi_launch_eltwise(&p, stream_) ? 5 : 0, s.note.c_str());
    break;
  }
  case Step::Reduce: {
    gcmi::ReduceParams p{};
    p.in = P(s.a), p.out = P(s.out), p.dt = s.a_dt, p.mean = s.mean;
    p.n_out = 1, p.n_red = 1;
    for (int d = 0; d < gcmi::ELT_MAX_RANK; d++)
      p.kdims[d] = p.rdims[d] = 1, p.kstr[d] = p.rstr[d] = 0;
    size_t pk = gcmi::ELT_MAX_RANK - s.kdims.size(), pr = gcmi::ELT_MAX_RANK - s.rdims.size();
    for (size_t d = 0; d < s.kdims.size(); d++)
      p.kdims[pk + d] = s.kdims[d], p.kstr[pk + d] = s.kstr[d], p.n_out *= s.kdims[d];
    for (size_t d = 0; d < s.rdims.size(); d++)
      p.rdims[pr + d] = s.rdims[d], p.rstr[pr + d] = s.rstr[d], p.n_red *= s.rdims[d];
    gc_check(gcmi_launch_reduce(&p, stream_) ? 5 : 0, s.note.c_str());
    break;
  }
  case Step::Fused: {
    gcmi::FusedParams p{};
    fill_fused_params(s, p);
    const size_t r = s.dims.size();
    const bool second_pass = s.row_end >= 0;
    for (int k = 0; k < p.n_in; k++)
      p.in[k] = P(s.f_in[(size_t)k]);
    p.out = P(s.out);
    // the furthest element any input index can reach lies inside its buffer, and the output fits
    auto esz = [](int dt) { return dt == GCMI_F32 ? 4 : 2; };
    for (int k = 0; k < p.n_in; k++) {
      int64_t far = 0;
      for (size_t d = 0; d < r; d++)
        far += (s.dims[d] - 1) * s.f_str[(size_t)k][d];
      if ((size_t)(far + 1) * (size_t)esz(p.in_dt[k]) > slots_[(size_t)s.f_in[(size_t)k]].bytes)
        throw std::runtime_error("fused group: an input index runs past its buffer (" + s.note + ")");
    }
    if ((size_t)(second_pass ? p.n : p.n / p.n_red) * (size_t)esz(p.out_dt) > slots_[(size_t)s.out].bytes)
      throw std::runtime_error("fused group: the result does not fit its buffer (" + s.note + ")");
    if (s.jit_fn) {
      bool aligned = (reinterpret_cast<uintptr_t>(p.out) & 15) == 0;
      for (int k = 0; k < p.n_in; k++)
        aligned = aligned && (reinterpret_cast<uintptr_t>(p.in[k]) & 15) == 0;
      if (aligned || !s.jit_vectors) {
        void *args[gcmi::FUSED_MAX_IN + 1];
        for (int k = 0; k < p.n_in; k++)
          args[k] = (void *)&p.in[k];
        args[p.n_in] = (void *)&p.out;
        hip_check(hipModuleLaunchKernel(s.jit_fn, s.jit_grid, 1, 1, s.jit_block, 1, 1, 0, stream_, args, nullptr), s.note.c_str());
        g_generated_launches++;
        break;
      }
    }
    gc_check(gcmi_launch_fused(&p, stream_) ? 5 : 0, s.note.c_str());
    break;
  }
  case Step::Softmax: {
    if (s.jit_fn) {
      const void *in = P(s.a);
      void *out = P(s.out);
      if (!s.jit_vectors || ((reinterpret_cast<uintptr_t>(in) | reinterpret_cast<uintptr_t>(out)) & 15) == 0) {
        void *args[2] = {(void *)&in, (void *)&out};
        hip_check(hipModuleLaunchKernel(s.jit_fn, s.jit_grid, 1, 1, s.jit_block, 1, 1, 0, stream_, args, nullptr), "SoftMax");
        g_generated_launches++;
        break;
      }
    }
    gcmi::SoftmaxParams p{};
    p.in = P(s.a), p.out = P(s.out), p.outer = s.outer, p.len = s.len, p.inner = s.inner, p.in_dt = s.a_dt, p.out_dt = s.out_dt;
    gc_check(gcmi_launch_softmax(&p, stream_) ? 5 : 0, "SoftMax");
    break;
  }
  }
}

// src/dnnl/dnnl_graph_compiler.cpp:64-103
void Executable::execute(dnnl_graph_compiler_tensor *inputs, dnnl_graph_compiler_tensor *outputs) {
  std::lock_guard<std::mutex> turn(run_mu_); // held until the stream has drained: the arena is this call's
  run(inputs, outputs, true);
}

// The launches of execute() on a stream of the caller's, in its order with the caller's other work there; nothing is
// waited for.  The executable's arena holds the intermediates, so calls on one executable must follow one another on
// one stream (or be ordered by the caller), and host buffers cannot take part.
void Executable::execute_async(dnnl_graph_compiler_tensor *inputs, dnnl_graph_compiler_tensor *outputs, hipStream_t stream) {
  for (const Step &s : steps_)
    if (s.kind == Step::Mha && s.scale_slot >= 0)
      throw std::invalid_argument("execute_async: the attention scale of this partition is a tensor that has to be read "
                                  "back to the host (a wait); use execute, or give the scale as a constant");
  std::lock_guard<std::mutex> turn(run_mu_);
  struct Swap {
    hipStream_t &slot, saved;
    Swap(hipStream_t &s, hipStream_t v) : slot(s), saved(s) { slot = v; }
    ~Swap() { slot = saved; }
  } swap(stream_, stream);
  run(inputs, outputs, false);
}

void Executable::run(dnnl_graph_compiler_tensor *inputs, dnnl_graph_compiler_tensor *outputs, bool wait) {
  auto find = [](dnnl_graph_compiler_tensor *ts, size_t n, size_t i, size_t id) -> dnnl_graph_compiler_tensor * {
    if (!ts)
      throw std::invalid_argument("Tensor not found");
    if (ts[i].id == id)
      return &ts[i];
    for (size_t j = 0; j < n; j++) // the order may differ from the argument order
      if (ts[j].id == id)
        return &ts[j];
    throw std::invalid_argument("Tensor not found");
  };
  for (size_t s = 0; s < slots_.size(); s++)
    ptr_[s] = slots_[s].staged ? nullptr : arena_ + slots_[s].offset;
  auto staged_ptr = [&](int slot) -> void * {
    const Slot &sl = slots_[(size_t)slot];
    return sl.staged ? (void *)(staging() + sl.offset) : (void *)(arena_ + sl.offset);
  };

  // inputs: device pointers are used in place, host buffers are staged
  for (size_t i = 0; i < g_.input_ids.size(); i++) {
    size_t id = g_.input_ids[i];
    auto *t = find(inputs, g_.input_ids.size(), i, id);
    if (t->ndims > DNNL_MAX_NDIMS)
      throw std::invalid_argument("Number of dimensions > DNNL_MAX_NDIMS");
    int slot = -1;
    for (size_t s = 0; s < slots_.size(); s++)
      if (slots_[s].is_input && slots_[s].tensor_id == (long)id)
        slot = (int)s;
    if (slot < 0)
      continue;
    if (!t->data) { // nothing to read: the kernels still get an address of the right size
      ptr_[(size_t)slot] = staged_ptr(slot);
      continue;
    }
    if (is_device_pointer(t->data)) {
      ptr_[(size_t)slot] = t->data;
    } else {
      if (!wait)
        throw std::invalid_argument("execute_async: input " + std::to_string(id) + " is not a device pointer");
      ptr_[(size_t)slot] = staged_ptr(slot);
      // a constant keeps its first contents: staged once
      const bool constant = g_.tensors.at(id).constant;
      if (const_staged_.size() < slots_.size())
        const_staged_.resize(slots_.size(), 0);
      if (constant && const_staged_[(size_t)slot])
        continue;
      hip_check(hipMemcpyAsync(ptr_[(size_t)slot], t->data, slots_[(size_t)slot].bytes, hipMemcpyHostToDevice, stream_), "stage input");
      const_staged_[(size_t)slot] = constant;
    }
  }
  std::vector<std::pair<void *, int>> copy_back;
  for (size_t i = 0; i < g_.output_ids.size(); i++) {
    size_t id = g_.output_ids[i];
    auto *t = find(outputs, g_.output_ids.size(), i, id);
    if (t->ndims > DNNL_MAX_NDIMS)
      throw std::invalid_argument("Number of dimensions > DNNL_MAX_NDIMS");
    int slot = slot_of_tensor_.at(id);
    if (!t->data)
      throw std::invalid_argument("Output tensor has no buffer");
    bool also_input = slots_[(size_t)slot].is_input;
    if (!wait && !is_device_pointer(t->data))
      throw std::invalid_argument("execute_async: output " + std::to_string(id) + " is not a device pointer");
    if (is_device_pointer(t->data) && !also_input && slots_[(size_t)slot].staged) {
      ptr_[(size_t)slot] = t->data;
    } else {
      if (!ptr_[(size_t)slot])
        ptr_[(size_t)slot] = staged_ptr(slot);
      copy_back.emplace_back(t->data, slot);
    }
  }
  if (step_done_.size() < steps_.size())
    step_done_.resize(steps_.size(), 0);
  // what an earlier call computed once (steps over constant tensors, column sums of constant weights) may still be
  // in flight on that call's stream
  if (once_recorded_ && once_stream_ != stream_)
    hip_check(hipStreamWaitEvent(stream_, once_done_, 0), "wait for constant results");
  for (size_t i = 0; i < steps_.size(); i++) {
    if (steps_[i].once && step_done_[i])
      continue;
    const bool keeps = steps_[i].once || (steps_[i].kind == Step::ColSum && steps_[i].op == 1 && !colsum_valid_[steps_[i].out]);
    launch(steps_[i]);
    step_done_[i] = steps_[i].once;
    if (keeps) { // record behind the last of them (re-recorded per step: cheap, and only in the first calls)
      if (!once_done_)
        hip_check(hipEventCreateWithFlags(&once_done_, hipEventDisableTiming), "hipEventCreate");
      hip_check(hipEventRecord(once_done_, stream_), "hipEventRecord");
      once_recorded_ = true, once_stream_ = stream_;
    }
  }
  for (auto &cb : copy_back) {
    hipMemcpyKind kind = is_device_pointer(cb.first) ? hipMemcpyDeviceToDevice : hipMemcpyDeviceToHost;
    hip_check(hipMemcpyAsync(cb.first, ptr_[(size_t)cb.second], slots_[(size_t)cb.second].bytes, kind, stream_), "copy result");
  }
  if (wait) {
    hip_check(hipStreamSynchronize(stream_), "execute");
    if (once_stream_ == stream_)
      once_recorded_ = false; // those results are final now: nobody has to wait for them again
  }
}

std::string Executable::describe() const {
  static const char *names[] = {"gemm_f32", "gemm_bf16", "gemm_int8", "colsum", "attention", "eltwise", "reduce", "softmax",
                                "fused", "attention mask"};
  std::ostringstream os;
  static const char *kernels[] = {"bounds-checked tile", "whole tiles, 8 waves", "whole tiles, 4 waves (one per SIMD)",
                                  "K slices + second pass", "weight streaming (+ second pass)",
                                  "small tiles, 4 waves, two workgroups per compute unit"};
  for (auto &s : steps_) {
    os << (s.kind == Step::Fused ? (s.sum_ins >= 0 ? "reduce" : "fused") : names[(int)s.kind]) << ": " << s.note << "\n";
    if ((s.kind == Step::GemmBf16 && s.batch <= 1 && !s.ta) || s.kind == Step::GemmInt8) {
      // the tile descriptor the launcher will choose for this shape (the counterpart of the reference's MatmulConfig)
      gcmi_gemm_tile_config c{};
      char why[160] = "";
      const int a_dt = s.kind == Step::GemmInt8 ? s.a_dt : GCMI_BF16;
      if (gcmi_gemm_tile_config_query(a_dt, s.M, s.N, s.K, s.tb ? 1 : 0, s.out_dt, s.mm_cfg.size() == 9 ? s.mm_cfg.data() : nullptr,
                                      &c, why, sizeof(why)) == 0) {
        os << "  tile: " << kernels[c.kernel] << ", " << c.bm << "x" << c.bn << " per workgroup, " << c.kbytes
           << " B of K per stage x " << c.stages << " stages, waves " << c.waves_m << "x" << c.waves_n << " of " << c.wave_m << "x"
           << c.wave_n << ", mfma " << c.mfma_m << "x" << c.mfma_n << "x" << c.mfma_k << ", split_k " << c.split_k << ", "
           << c.workgroups << " workgroups";
        if (c.split_k > 1) // the slot the partial sums of the slices were planned into
          os << ", workspace " << (s.ws >= 0 ? slots_[(size_t)s.ws].bytes : 0) << " B";
        if (c.from_attrs)
          os << " [MatmulConfig attributes applied]";
        else if (why[0])
          os << " [" << why << "]";
        else if (s.mm_cfg.size() == 9)
          os << " [MatmulConfig attributes leave the default]";
        os << "\n";
      }
    }
  }
  if (!g_.target_hints.empty()) {
    os << "target hints (CPU, not used):";
    for (auto &h : g_.target_hints)
      os << " " << h.first << "=" << h.second;
    os << "\n";
  }
  os << "arena: " << arena_bytes_ << " bytes (" << arena_bytes_no_reuse_ << " with one region per buffer); staging for host buffers: "
     << staging_bytes_ << " bytes, allocated by the first execute that passes one\n";
  return os.str();
}

} // namespace gcapi
