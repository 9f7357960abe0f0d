// bf16 x bf16 -> f32 GEMMs: the 256x256 MFMA tile kernels (gemm_tile256.hpp) and the streaming kernels for a short
// A against [N,K] weights (gemm_rows32.hpp: up to 32 rows; gemm_skinny.hpp: up to 64 rows where a caller's slice
// count asks for it, and the shapes the former does not take).
#include "gemm_rows32.hpp"
#include "gemm_skinny.hpp"

extern "C" int gcmi_launch_gemm_bf16(const gcmi::GemmParams *p, hipStream_t stream) {
  int rc = gcmi::launch_rows32(p, stream);
  if (rc >= 0)
    return rc;
  rc = gcmi::launch_skinny_nt(p, stream);
  if (rc >= 0)
    return rc;
  return gcmi::launch_tile256<2>(p, stream);
}

// floats of workspace (GemmParams::partial) the launch above would use for this call: 0 when K is not sliced
extern "C" int64_t gcmi_launch_gemm_bf16_workspace(const gcmi::GemmParams *p) {
  int64_t want = 0;
  if (gcmi::launch_rows32(p, nullptr, &want) >= 0)
    return want;
  if (gcmi::launch_skinny_nt(p, nullptr, &want) >= 0)
    return want;
  gcmi::launch_tile256<2>(p, nullptr, &want);
  return want;
}

// what the launch above would choose (nothing is launched)
extern "C" int gcmi_launch_gemm_bf16_config(const gcmi::GemmParams *p, gcmi::GemmTileConfig *cfg) {
  if (gcmi::launch_rows32(p, (hipStream_t)-1, nullptr, cfg) >= 0)
    return 0;
  if (gcmi::launch_skinny_nt(p, (hipStream_t)-1, nullptr, cfg) >= 0)
    return 0;
  return gcmi::launch_tile256<2>(p, (hipStream_t)-1, nullptr, cfg);
}

// Scratch of the entry point that allocates nothing (gcmi_gemm_bf16_noalloc): the partial sums of K-sliced calls.
// Each device the library runs on holds its own copy until the process ends.  `scratch` is only a host-side
// stand-in here: its device address is asked for once per device and kept.
static constexpr size_t GCMI_NOALLOC_SCRATCH_BYTES = (size_t)32 << 20;
static __device__ __align__(256) unsigned char scratch[GCMI_NOALLOC_SCRATCH_BYTES];

extern "C" int gcmi_noalloc_scratch(void **ptr, size_t *bytes) {
  static void *dev_ptr[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
    return 5;
  void *q = __atomic_load_n(&dev_ptr[dev], __ATOMIC_ACQUIRE);
  if (!q) {
    if (hipGetSymbolAddress(&q, HIP_SYMBOL(scratch)) != hipSuccess || !q)
      return 5;
    __atomic_store_n(&dev_ptr[dev], q, __ATOMIC_RELEASE); // the same value from every thread that gets here
  }
  *ptr = q;
  *bytes = GCMI_NOALLOC_SCRATCH_BYTES;
  return 0;
}
