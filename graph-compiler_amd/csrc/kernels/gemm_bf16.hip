// bf16 x bf16 -> f32 GEMMs: the 256x256 MFMA tile kernels (gemm_tile256.hpp) and the streaming kernel for a short
// A against [N,K] weights (gemm_skinny.hpp).
#include "gemm_skinny.hpp"

extern "C" int gcmi_launch_gemm_bf16(const gcmi::GemmParams *p, hipStream_t stream) {
  const int rc = gcmi::launch_skinny_nt(p, stream);
  if (rc >= 0)
    return rc;
  return gcmi::launch_tile256<2>(p, stream);
}
