// Kernel launch of the library's device code: an ordinary launch, or, when the calling thread has left a pair
// of events with rt_time_next_launch, a launch that writes the dispatch's own start and end timestamps into
// them (what a profiler reports as the kernel's duration; a pair of hipEventRecord calls around a launch also
// counts the gaps to the neighbouring kernels, several microseconds on this part).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_ext.h>

#include "rt_common.h"

#define RT_LAUNCH(kernel, grid, block, shmem, stream, ...)                                              \
  do {                                                                                                  \
    const rt::LaunchEvents rt_ev_ = rt::take_launch_events();                                           \
    if (rt_ev_.start || rt_ev_.stop)                                                                    \
      hipExtLaunchKernelGGL(kernel, grid, block, shmem, stream, static_cast<hipEvent_t>(rt_ev_.start),  \
                            static_cast<hipEvent_t>(rt_ev_.stop), 0, __VA_ARGS__);                      \
    else                                                                                                \
      hipLaunchKernelGGL(kernel, grid, block, shmem, stream, __VA_ARGS__);                              \
  } while (0)
