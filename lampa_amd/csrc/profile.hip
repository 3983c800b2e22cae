// Per-kernel timing of the library's own launches with HIP events recorded on the launch stream.
// A profiling aid for the benchmark: one recording at a time, not thread-safe, adds a few event records per call.
#include "common.h"

#include <string.h>

#define PROF_MAX 4096

static bool g_recording = false;
static int g_count = 0;
static hipEvent_t g_events[PROF_MAX];
static const char* g_names[PROF_MAX];

bool lampa_prof_recording() { return g_recording; }

void lampa_prof_mark(hipStream_t stream, const char* name) {
  if (!g_recording || g_count >= PROF_MAX) return;
  if (hipEventCreate(&g_events[g_count]) != hipSuccess) return;
  (void)hipEventRecord(g_events[g_count], stream);
  g_names[g_count] = name;
  ++g_count;
}

// Starts recording the kernels launched by subsequent library calls (on whatever stream they use).
extern "C" int lampa_profile_begin() {
  if (g_recording) return LAMPA_ERR_INVALID;
  g_count = 0;
  g_recording = true;
  return LAMPA_OK;
}

// Stops recording, waits for the recorded work and returns the number of kernel intervals n (<= max_entries):
// ms[i] is the time between the previous mark and the mark after kernel i, names[i] points to a static string.
extern "C" int lampa_profile_end(int max_entries, float* ms, const char** names) {
  if (!g_recording) return LAMPA_ERR_INVALID;
  g_recording = false;
  int n = 0;
  if (g_count > 0) (void)hipEventSynchronize(g_events[g_count - 1]);
  for (int i = 1; i < g_count; ++i) {
    if (strcmp(g_names[i], "start") == 0) continue;
    float t = 0.0f;
    (void)hipEventElapsedTime(&t, g_events[i - 1], g_events[i]);
    if (n < max_entries) {
      if (ms) ms[n] = t;
      if (names) names[n] = g_names[i];
      ++n;
    }
  }
  for (int i = 0; i < g_count; ++i) (void)hipEventDestroy(g_events[i]);
  g_count = 0;
  return n;
}
