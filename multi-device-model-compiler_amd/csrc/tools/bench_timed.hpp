// The timed region shared by the launch loops and the ceiling probes of bench.py:
// `warmup` untimed launches, then `steps` launches between two events recorded on the
// launch stream.  Measurement plumbing only.
#pragma once
#include <hip/hip_runtime.h>

namespace mgpu_bench {

// The rotation through a caller's buffer sets never restarts: the index handed to
// launch() keeps counting through the warm-up launches, the timed launches and every
// later region of the process, so a timed launch always meets the set that has gone
// untouched the longest.  (A loop that began again at set 0 after its warm-up would find
// the sets the warm-up had just used still in the Infinity Cache.)
inline unsigned long rotation = 0;

template <typename F> float timed(F &&launch, int steps, int warmup, hipStream_t stream) {
  for (int i = 0; i < warmup; i++) launch(rotation++);
  if (hipStreamSynchronize(stream) != hipSuccess) return -1.0f;
  hipEvent_t e0, e1;
  if (hipEventCreate(&e0) != hipSuccess || hipEventCreate(&e1) != hipSuccess) return -1.0f;
  (void)hipEventRecord(e0, stream);
  for (int i = 0; i < steps; i++) launch(rotation++);
  (void)hipEventRecord(e1, stream);
  float ms = -1.0f;
  if (hipEventSynchronize(e1) != hipSuccess || hipEventElapsedTime(&ms, e0, e1) != hipSuccess) ms = -1.0f;
  (void)hipEventDestroy(e0);
  (void)hipEventDestroy(e1);
  return hipGetLastError() == hipSuccess ? ms : -1.0f;
}

} // namespace mgpu_bench
