// Function-space qualifiers for the CuSync headers.
//
// The host half of the API (constructing stages, pairing them, launching the
// wait kernel) must compile with a plain C++ compiler; the device half
// (tile / wait / post) only exists when the translation unit is compiled by
// hipcc.  Same role as the macro header of the reference
// (src/include/cusync/cusync_defines.h:4-26).
#pragma once

#if defined(__HIPCC__)
  #include <hip/hip_runtime.h>
  #define CUSYNC_DEVICE __device__ __forceinline__
  #define CUSYNC_HOST __host__ __forceinline__
  #define CUSYNC_DEVICE_HOST __device__ __host__ __forceinline__
  #define CUSYNC_GLOBAL __global__
  #define CUSYNC_HAS_DEVICE 1
#else
  #define CUSYNC_DEVICE inline
  #define CUSYNC_HOST inline
  #define CUSYNC_DEVICE_HOST inline
  #define CUSYNC_GLOBAL
  #define CUSYNC_HAS_DEVICE 0
  // Minimal dim3 so host-only translation units see the same type name.
  #ifndef CUSYNC_DIM3_DEFINED
  #define CUSYNC_DIM3_DEFINED
  struct dim3 {
    unsigned int x, y, z;
    constexpr dim3(unsigned int x_ = 1, unsigned int y_ = 1, unsigned int z_ = 1) : x(x_), y(y_), z(z_) {}
  };
  #endif
#endif
