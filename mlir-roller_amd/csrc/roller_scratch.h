// Internal to libroller_hip.so: the fixed device-memory scratch array behind rl_gemm_plan_launch_static.
#ifndef ROLLER_SCRATCH_H
#define ROLLER_SCRATCH_H

#include <hip/hip_runtime_api.h>

// 256 KiB of arrival counters (65536 tiles) + 64 MiB of slots for the pieces of split tiles
#define RL_STATIC_SCRATCH_COUNTER_BYTES (256u * 1024u)
#define RL_STATIC_SCRATCH_BYTES (RL_STATIC_SCRATCH_COUNTER_BYTES + 64u * 1024u * 1024u)

extern "C" hipError_t rl_scratch_setup(int device);
extern "C" void* rl_scratch_address(int device);
extern "C" hipError_t rl_scratch_zero_c(float* C, int ldc, int M, int N, hipStream_t stream);

#endif
