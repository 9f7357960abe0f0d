// hiprtc front: source -> code object -> loaded module (see fused_jit.h).
#include "fused_jit.h"

#include <hip/hip_runtime_api.h>
#include <hip/hiprtc.h>

#include <deque>
#include <map>
#include <mutex>

namespace gcjit {
namespace {

// the text of kernels/op_codes.h and kernels/device_math.hpp, written out by the build as one raw string literal
const char kSharedText[] =
#include "jit_prelude.inc"
    ;

const char kTypes[] =
    "typedef unsigned short uint16_t;\ntypedef unsigned int uint32_t;\ntypedef long long int64_t;\n"
    "typedef unsigned long long uint64_t;\ntypedef float f4_ __attribute__((ext_vector_type(4)));\n"
    "typedef unsigned u2_ __attribute__((ext_vector_type(2)));\n";

std::string full_source(const std::vector<FusedKernelSource> &kernels) {
  std::string s = Module::prelude();
  for (const FusedKernelSource &k : kernels)
    s += "\n" + k.source;
  return s;
}

// Packed-f32 VALU forms stay switched off, as in the kernels built with the library.
bool compile(const std::string &src, const std::string &arch, std::vector<char> &code, std::string &log) {
  hiprtcProgram prog = nullptr;
  if (hiprtcCreateProgram(&prog, src.c_str(), "fused_groups.hip", 0, nullptr, nullptr) != HIPRTC_SUCCESS) {
    log = "hiprtcCreateProgram failed";
    return false;
  }
  const std::string arch_opt = "--offload-arch=" + arch;
  const char *opts[] = {arch_opt.c_str(), "-O3", "-std=c++17", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
  const hiprtcResult rc = hiprtcCompileProgram(prog, (int)(sizeof(opts) / sizeof(opts[0])), opts);
  size_t n = 0;
  if (hiprtcGetProgramLogSize(prog, &n) == HIPRTC_SUCCESS && n > 1) {
    log.resize(n);
    (void)hiprtcGetProgramLog(prog, &log[0]);
  }
  bool ok = rc == HIPRTC_SUCCESS;
  if (ok) {
    ok = hiprtcGetCodeSize(prog, &n) == HIPRTC_SUCCESS && n > 0;
    if (ok) {
      code.resize(n);
      ok = hiprtcGetCode(prog, code.data()) == HIPRTC_SUCCESS;
    }
  } else if (log.empty()) {
    log = hiprtcGetErrorString(rc);
  }
  (void)hiprtcDestroyProgram(&prog);
  return ok;
}

std::mutex g_mu;
// "<device>|<source>" -> module.  The map holds weak references: a module is unloaded when the last executable
// that uses it goes away and it has dropped out of the short list of recently built ones (kept so that compiling
// the same partition again right after destroying it does not cost another run of the compiler).  Neither
// container is ever destroyed: modules must not be unloaded during static destruction, when the HIP runtime may
// already be gone.
constexpr size_t kRecentModules = 32;
std::map<std::string, std::weak_ptr<Module>> &cache() {
  static auto *c = new std::map<std::string, std::weak_ptr<Module>>();
  return *c;
}
std::deque<std::shared_ptr<Module>> &recent() {
  static auto *r = new std::deque<std::shared_ptr<Module>>();
  return *r;
}
void remember(const std::shared_ptr<Module> &m) { // g_mu held
  auto &r = recent();
  for (auto it = r.begin(); it != r.end(); ++it)
    if (*it == m) {
      r.erase(it);
      break;
    }
  r.push_back(m);
  while (r.size() > kRecentModules)
    r.pop_front();
}

} // namespace

const char *Module::prelude() {
  static const std::string text = std::string(kTypes) + kSharedText;
  return text.c_str();
}

Module::~Module() {
  if (mod_)
    (void)hipModuleUnload(mod_);
}

hipFunction_t Module::function(const std::string &name) const {
  hipFunction_t f = nullptr;
  if (!mod_ || hipModuleGetFunction(&f, mod_, name.c_str()) != hipSuccess)
    return nullptr;
  return f;
}

std::shared_ptr<Module> Module::build(const std::vector<FusedKernelSource> &kernels, std::string &error) {
  int dev = 0;
  hipDeviceProp_t prop;
  if (hipGetDevice(&dev) != hipSuccess || hipGetDeviceProperties(&prop, dev) != hipSuccess) {
    error = "no current device";
    return nullptr;
  }
  const std::string src = full_source(kernels), key = std::to_string(dev) + "|" + src;
  std::lock_guard<std::mutex> lock(g_mu);
  auto it = cache().find(key);
  if (it != cache().end()) {
    if (auto alive = it->second.lock()) {
      remember(alive);
      return alive;
    }
    cache().erase(it);
  }
  std::vector<char> code;
  if (!compile(src, prop.gcnArchName, code, error))
    return nullptr;
  std::shared_ptr<Module> m(new Module());
  if (hipModuleLoadData(&m->mod_, code.data()) != hipSuccess) {
    (void)hipGetLastError();
    error = "hipModuleLoadData failed";
    return nullptr;
  }
  for (auto e = cache().begin(); e != cache().end();) // entries whose module is gone
    e = e->second.expired() ? cache().erase(e) : std::next(e);
  cache()[key] = m;
  remember(m);
  return m;
}

std::string compile_only(const std::vector<FusedKernelSource> &kernels, const std::string &arch) {
  std::vector<char> code;
  std::string log;
  if (compile(full_source(kernels), arch, code, log))
    return "";
  return log.empty() ? "compilation failed" : log;
}

} // namespace gcjit
