// Host stand-in for <hip/hip_runtime.h>, used ONLY by tests: it lets the
// library's unchanged source be compiled for the CPU so that every kernel's
// indexing can be checked under AddressSanitizer and compared with the oracle
// without a GPU.  A launch runs the kernel once per (workgroup, thread) in
// sequence (grids of one or two dimensions); that is exact for these kernels because they use no LDS, no
// barriers and no cross-thread communication.  Never part of the product.
#pragma once
#include <cstdint>
#include <cstring>

#define __global__
#define __device__
#define __host__
#define __forceinline__ inline __attribute__((always_inline))
#define __launch_bounds__(...)

struct dim3 {
  unsigned x, y, z;
  constexpr dim3(unsigned x_ = 1, unsigned y_ = 1, unsigned z_ = 1) : x(x_), y(y_), z(z_) {}
};

inline thread_local dim3 threadIdx, blockIdx, blockDim, gridDim;

typedef void* hipStream_t;
typedef int hipError_t;
constexpr hipError_t hipSuccess = 0;
inline hipError_t hipGetLastError() { return hipSuccess; }
inline const char* hipGetErrorString(hipError_t) { return "emulated"; }

// a "device" array is ordinary host memory here; its symbol is its address
#define __align__(n) __attribute__((aligned(n)))
#define HIP_SYMBOL(x) (x)
inline hipError_t hipGetDevice(int* dev) { *dev = 0; return hipSuccess; }
inline hipError_t hipGetSymbolAddress(void** ptr, const void* symbol) { *ptr = const_cast<void*>(symbol); return hipSuccess; }

inline uint32_t __float_as_uint(float f) { uint32_t u; std::memcpy(&u, &f, 4); return u; }
inline float __uint_as_float(uint32_t u) { float f; std::memcpy(&f, &u, 4); return f; }

#define hipLaunchKernelGGL(kernel, grid, block, shmem, stream, ...)      \
  do {                                                                   \
    (void)(stream);                                                      \
    gridDim = (grid);                                                    \
    blockDim = (block);                                                  \
    for (unsigned by_ = 0; by_ < gridDim.y; ++by_)                       \
      for (unsigned bx_ = 0; bx_ < gridDim.x; ++bx_)                     \
        for (unsigned tx_ = 0; tx_ < blockDim.x; ++tx_) {                \
          blockIdx = dim3(bx_, by_, 0);                                  \
          threadIdx = dim3(tx_, 0, 0);                                   \
          kernel(__VA_ARGS__);                                           \
        }                                                                \
  } while (0)

// the library's launch macro: no status to collect here
#define PCCL_LAUNCH(kernel, grid, block, shmem, stream, ...) hipLaunchKernelGGL(kernel, grid, block, shmem, stream, __VA_ARGS__)
