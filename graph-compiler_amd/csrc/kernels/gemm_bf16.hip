// bf16 x bf16 -> f32 GEMMs: the 256x256 MFMA tile kernels (gemm_tile256.hpp) and the streaming kernel for a short
// A against [N,K] weights (gemm_skinny.hpp).
#include "gemm_skinny.hpp"

extern "C" int gcmi_launch_gemm_bf16(const gcmi::GemmParams *p, hipStream_t stream) {
  const int rc = gcmi::launch_skinny_nt(p, stream);
  if (rc >= 0)
    return rc;
  return gcmi::launch_tile256<2>(p, stream);
}

// floats of workspace (GemmParams::partial) the launch above would use for this call: 0 when K is not sliced
extern "C" int64_t gcmi_launch_gemm_bf16_workspace(const gcmi::GemmParams *p) {
  int64_t want = 0;
  if (gcmi::launch_skinny_nt(p, nullptr, &want) >= 0)
    return want;
  gcmi::launch_tile256<2>(p, nullptr, &want);
  return want;
}
