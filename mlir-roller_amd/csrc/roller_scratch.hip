// The one piece of libroller_hip.so that is device code: a fixed scratch array in device memory for
// rl_gemm_plan_launch_static, the launch entry point that allocates nothing.  Everything else in the
// library is host code that JIT-compiles its kernels; this file exists so that a stream-K launch has
// a workspace that was never hipMalloc'ed -- it is part of the library's own code object and lives
// on every GPU the library's code is loaded on until the process ends.
#include <hip/hip_runtime.h>

#include "roller_scratch.h"

// arrival counters (zero when the code object is loaded; every kernel leaves them at zero), then the slots
static __device__ __align__(256) unsigned char scratch[RL_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];   // device address of `scratch` on each device, set by rl_scratch_setup
}  // namespace

// Looks up where `scratch` lives on `device`, which must be the calling thread's current device
// (the array's name is a host-side handle, not an address: every GPU has its own copy at its own
// address).  Called once per device from rl_init.
extern "C" __attribute__((visibility("hidden"))) hipError_t rl_scratch_setup(int device) {
  if (device < 0 || device >= kMaxDevices) return hipErrorInvalidDevice;
  void* ptr = nullptr;
  const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
  if (e != hipSuccess) return e;
  g_scratch_ptr[device] = ptr;
  return hipSuccess;
}

// Device address of the scratch array on `device` (NULL before rl_scratch_setup).
extern "C" __attribute__((visibility("hidden"))) void* rl_scratch_address(int device) {
  return device >= 0 && device < kMaxDevices ? g_scratch_ptr[device] : nullptr;
}

// C[0..M)[0..N) = 0 for a row-major C with leading dimension ldc: what a stream-K launch with K == 0
// comes down to.  A kernel rather than a memset call, so that it may sit in a captured graph.
static __global__ void zero_rows(float* __restrict__ C, long ldc, int M, int N) {
  const long n = (long)M * N;
  for (long i = blockIdx.x * (long)blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) C[(i / N) * ldc + i % N] = 0.0f;
}

extern "C" __attribute__((visibility("hidden"))) hipError_t rl_scratch_zero_c(float* C, int ldc, int M, int N, hipStream_t stream) {
  const long n = (long)M * N;
  const unsigned blocks = (unsigned)((n + 255) / 256 < 4096 ? (n + 255) / 256 : 4096);
  hipLaunchKernelGGL(zero_rows, dim3(blocks ? blocks : 1), dim3(256), 0, stream, C, (long)ldc, M, N);
  return hipGetLastError();
}
