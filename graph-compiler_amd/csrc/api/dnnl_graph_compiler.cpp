// The six C entry points of the oneDNN-Graph compiler backend
// (src/dnnl/dnnl_graph_compiler.cpp:157-226 of intel/graph-compiler) and the
// inert gc-c registration shims.  No exception crosses the ABI; the mapping of
// exception classes to dnnl_status_t is the reference's (:172-182, 193-206,
// 217-225): invalid_argument -> invalid_graph, logic_error -> unimplemented,
// bad_alloc -> out_of_memory, anything else -> runtime_error; during execute
// everything but bad_alloc is a runtime_error.
#include <cstdio>
#include <cstring>
#include <new>
#include <stdexcept>
#include <string>

#include "dnnl_graph_compiler.h"
#include "executable.h"
#include "gc-c/Dialects.h"
#include "gc-c/Passes.h"
#include "gc_hip_kernels.h"
#include "mlir_text.h"

struct dnnl_graph_compiler {
  uint32_t num_threads = 0;
  int device = 0;
};

struct dnnl_graph_compiler_executable {
  gcapi::Executable impl;
  explicit dnnl_graph_compiler_executable(const char *json) : impl(json) {}
  explicit dnnl_graph_compiler_executable(gcapi::Graph g) : impl(std::move(g)) {}
};

namespace {
thread_local std::string g_last_error;
void remember(const char *what) {
  g_last_error = what ? what : "";
  if (getenv("GC_DEBUG"))
    fprintf(stderr, "[graph-compiler] %s\n", g_last_error.c_str());
}
} // namespace

extern "C" const char *dnnl_graph_compiler_last_error(void) { return g_last_error.c_str(); }

// No exception crosses the C ABI.  The mapping of the reference (src/dnnl/dnnl_graph_compiler.cpp:190-226): bad
// input -> invalid_graph (compile) / invalid_arguments (execute), unsupported -> unimplemented, bad_alloc ->
// out_of_memory, anything else -> runtime_error.
namespace {
template <typename F> dnnl_status_t guarded(dnnl_status_t on_invalid_argument, F &&body) {
  try {
    body();
    return dnnl_success;
  } catch (const std::invalid_argument &e) {
    remember(e.what());
    return on_invalid_argument;
  } catch (const std::logic_error &e) {
    remember(e.what());
    return dnnl_unimplemented;
  } catch (const std::bad_alloc &) {
    remember("out of memory");
    return dnnl_out_of_memory;
  } catch (const std::exception &e) {
    remember(e.what());
    return dnnl_runtime_error;
  } catch (...) {
    remember("unknown error");
    return dnnl_runtime_error;
  }
}
void copy_out(const std::string &d, char *buf, size_t len) {
  if (buf && len) {
    const size_t n = d.size() < len - 1 ? d.size() : len - 1;
    memcpy(buf, d.data(), n);
    buf[n] = 0;
  }
}
} // namespace

extern "C" const dnnl_graph_compiler_version *dnnl_graph_compiler_get_version(void) {
  static const dnnl_graph_compiler_version ver = {
      {DNNL_GC_API_V_MAJOR, DNNL_GC_API_V_MINOR, DNNL_GC_API_V_PATCH, DNNL_GC_API_V_HASH}, // API version (oneDNN's)
      {0, 1, 0, "gfx950"}};                                                               // this library's own
  return &ver;
}

extern "C" dnnl_status_t dnnl_graph_compiler_create(const dnnl_graph_compiler_context *ctx, const dnnl_graph_compiler **gc) {
  if (!gc)
    return dnnl_invalid_arguments;
  try {
    auto *c = new dnnl_graph_compiler();
    c->num_threads = ctx ? ctx->num_threads : 0;
    *gc = c;
    return dnnl_success;
  } catch (const std::bad_alloc &) {
    return dnnl_out_of_memory;
  } catch (...) {
    return dnnl_runtime_error;
  }
}

extern "C" void dnnl_graph_compiler_destroy(const dnnl_graph_compiler *gc) { delete gc; }

extern "C" dnnl_status_t dnnl_graph_compiler_compile(const dnnl_graph_compiler *gc, const char *graph_json,
                                                     const dnnl_graph_compiler_executable **exe) {
  if (!gc || !exe)
    return dnnl_invalid_arguments;
  return guarded(dnnl_invalid_graph, [&] { *exe = new dnnl_graph_compiler_executable(graph_json); });
}

// The same for a module in MLIR's textual form (what the reference's gc-cpu-runner and benchgc's
// `--driver mlir` take, test/benchgc/cases/*.mlir); see mlir_text.h for the accepted subset.
extern "C" dnnl_status_t dnnl_graph_compiler_compile_mlir(const dnnl_graph_compiler *gc, const char *module_text,
                                                          const dnnl_graph_compiler_executable **exe) {
  if (!gc || !exe)
    return dnnl_invalid_arguments;
  return guarded(dnnl_invalid_graph, [&] { *exe = new dnnl_graph_compiler_executable(gcapi::parse_mlir(module_text)); });
}

extern "C" void dnnl_graph_compiler_destroy_executable(const dnnl_graph_compiler_executable *exe) { delete exe; }

extern "C" dnnl_status_t dnnl_graph_compiler_execute(const dnnl_graph_compiler_executable *exe,
                                                     dnnl_graph_compiler_tensor *inputs,
                                                     dnnl_graph_compiler_tensor *outputs) {
  if (!exe)
    return dnnl_invalid_arguments;
  // like the reference's, this may be called from several threads; calls on one executable take turns inside.
  // A missing tensor is a runtime error here, as there (the reference's execute maps every exception to it, :214-226)
  return guarded(dnnl_runtime_error,
                 [&] { const_cast<dnnl_graph_compiler_executable *>(exe)->impl.execute(inputs, outputs); });
}

extern "C" dnnl_status_t dnnl_graph_compiler_execute_async(const dnnl_graph_compiler_executable *exe,
                                                           dnnl_graph_compiler_tensor *inputs,
                                                           dnnl_graph_compiler_tensor *outputs, void *stream) {
  if (!exe)
    return dnnl_invalid_arguments;
  return guarded(dnnl_invalid_arguments, [&] {
    const_cast<dnnl_graph_compiler_executable *>(exe)->impl.execute_async(inputs, outputs, (hipStream_t)stream);
  });
}

// Parse, verify and plan a partition without touching the GPU; writes the
// launch plan into buf and returns the status compile would have returned for
// the host-side stages.
extern "C" dnnl_status_t dnnl_graph_compiler_explain(const char *graph_json, char *buf, size_t len) {
  return guarded(dnnl_invalid_graph, [&] { copy_out(gcapi::Executable(graph_json, true).describe(), buf, len); });
}

extern "C" dnnl_status_t dnnl_graph_compiler_explain_mlir(const char *module_text, char *buf, size_t len) {
  return guarded(dnnl_invalid_graph,
                 [&] { copy_out(gcapi::Executable(gcapi::parse_mlir(module_text), true).describe(), buf, len); });
}

extern "C" dnnl_status_t dnnl_graph_compiler_generated_source_mlir(const char *module_text, const char *check_arch, char *buf,
                                                                   size_t len) {
  return guarded(dnnl_invalid_graph, [&] {
    gcapi::Executable e(gcapi::parse_mlir(module_text), true);
    const std::vector<gcjit::FusedKernelSource> ks = e.generated_kernels();
    std::string d;
    for (const auto &k : ks)
      d += k.source + "\n";
    copy_out(d, buf, len);
    if (check_arch && !ks.empty()) {
      const std::string log = gcjit::compile_only(ks, check_arch);
      if (!log.empty())
        throw std::runtime_error(log);
    }
  });
}

extern "C" long dnnl_graph_compiler_generated_kernel_launches(void) { return gcapi::Executable::generated_launches(); }

// gc-c shims
extern "C" MlirDialectHandle mlirGetDialectHandle__onednn_graph__(void) { return MlirDialectHandle{nullptr}; }
extern "C" MlirDialectHandle mlirGetDialectHandle__cpuruntime__(void) { return MlirDialectHandle{nullptr}; }
extern "C" void mlirRegisterAllGCPassesAndPipelines(void) {}
