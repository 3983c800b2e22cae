// Shared helpers for the gfx950 kernels of the LSH + gated-delta path.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#define LAMPA_OK 0
#define LAMPA_ERR_INVALID (-1)      // bad argument (null pointer, size, unsupported combination)
#define LAMPA_ERR_WORKSPACE (-2)    // workspace missing or too small
#define LAMPA_ERR_LAUNCH (-3)       // HIP reported an error at launch
#define LAMPA_ERR_UNSUPPORTED (-4)  // shape or dtype outside what the kernels are built for

static inline int lampa_launch_status() {
  hipError_t e = hipGetLastError();
  return e == hipSuccess ? LAMPA_OK : LAMPA_ERR_LAUNCH;
}

static inline int64_t lampa_align_up(int64_t x, int64_t a) { return (x + a - 1) / a * a; }

__device__ __forceinline__ int lane_id() { return threadIdx.x & 63; }

// Optional per-kernel timing with HIP events on the launch stream (see profile.hip). No-ops unless a
// recording is open; the launchers call LAMPA_PROF(stream, "start") first and LAMPA_PROF(stream, "<kernel>") after
// each launch.
void lampa_prof_mark(hipStream_t stream, const char* name);
bool lampa_prof_recording();  // a recording is open: launchers keep everything on the caller's stream then
#define LAMPA_PROF(stream, name) lampa_prof_mark((stream), (name))
