// Shader-clock probe (a measurement aid; see kmoe_clock_probe in kmoe.h).
//
// One wave per workgroup alternates between two runs of FIXED length in shader clocks - a run of s_sleep
// instructions and a chain of dependent v_fma_f32 - and stamps each run with the constant 100 MHz counter
// (s_memrealtime) and with s_memtime. Launched on a second stream beside a kernel under test it answers two
// questions at once: whether s_memtime follows the shader clock (the ticks of a run stay constant whatever the
// load, while its duration by the 100 MHz counter stretches), and what that clock is (ticks / duration).
#include <hip/hip_runtime.h>

#include "kmoe_common.h"

namespace kmoe {
namespace {

constexpr int kSleepsPerRun = 8;     // x s_sleep 127 (64 x 127 clocks each)
constexpr int kFmaPerRun = 64 * 32;  // dependent v_fma_f32 per run

__global__ __launch_bounds__(64) void clock_probe_kernel(long long* samples, int reps) {
  float a = threadIdx.x * 1e-9f;
  const float b = 1.0000001f;
  for (int r = 0; r < reps; ++r) {
    const long long t0 = wall_clock64(), c0 = clock64();
    if (r & 1) {
#pragma unroll
      for (int i = 0; i < kSleepsPerRun; ++i) asm volatile("s_sleep 127" ::: "memory");
    } else {
      for (int i = 0; i < kFmaPerRun / 32; ++i) {
#pragma unroll
        for (int j = 0; j < 32; ++j) asm volatile("v_fma_f32 %0, %0, %1, %1" : "+v"(a) : "v"(b));
      }
    }
    const long long t1 = wall_clock64(), c1 = clock64();
    if (threadIdx.x == 0) {
      long long* o = samples + (static_cast<size_t>(blockIdx.x) * reps + r) * 3;
      o[0] = t0;
      o[1] = t1 - t0;
      o[2] = c1 - c0;
    }
  }
  if (a == 12345.678f) samples[0] = 0;  // keeps the chain alive
}

}  // namespace
}  // namespace kmoe

extern "C" int kmoe_clock_probe(int64_t* samples, int n_workgroups, int reps, kmoe_stream_t stream) {
  using namespace kmoe;
  const char* what = "kmoe_clock_probe";
  KMOE_REQUIRE(samples != nullptr, KMOE_ERR_NULL, "%s: samples is NULL", what);
  KMOE_REQUIRE(n_workgroups >= 1 && n_workgroups <= 64 && reps >= 2 && reps <= (1 << 20), KMOE_ERR_SHAPE,
               "%s: n_workgroups %d (1..64), reps %d (2..1048576)", what, n_workgroups, reps);
  hipLaunchKernelGGL(clock_probe_kernel, dim3(n_workgroups), dim3(64), 0, static_cast<hipStream_t>(stream),
                     reinterpret_cast<long long*>(samples), reps);
  return check_launch(what);
}
