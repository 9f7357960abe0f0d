// bf16 x bf16 -> f32 instantiation of the 256x256 MFMA GEMM (see gemm_tile256.hpp).
#include "gemm_tile256.hpp"

extern "C" int gcmi_launch_gemm_bf16(const gcmi::GemmParams *p, hipStream_t stream) {
  return gcmi::launch_tile256<2>(p, stream);
}
