// Shared device-side vocabulary for the gfx950 kernels: vector types, bf16
// rounding, post-op (epilogue) math.  Wave size is 64 throughout.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace gcmi {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef float f32x16_t __attribute__((ext_vector_type(16)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x16_t __attribute__((ext_vector_type(16)));
typedef int i32x4_t __attribute__((ext_vector_type(4)));
typedef int i32x2_t __attribute__((ext_vector_type(2)));
typedef unsigned short u16x4_t __attribute__((ext_vector_type(4)));

#define GCMI_LDS __attribute__((address_space(3)))

} // namespace gcmi

#include "op_codes.h"
#include "device_math.hpp"

// compute units of the current device (host side, cached per device)
static inline int gcmi_num_cus() {
  static int cache[64];
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
    return 256;
  if (cache[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      n = 256;
    cache[dev] = n;
  }
  return cache[dev];
}
