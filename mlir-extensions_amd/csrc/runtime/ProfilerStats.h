// Statistics over per-launch kernel times, as printed by the profiling loop of
// gpuLaunchKernel.  Formulas follow
// lib/ExecutionEngine/ExecutionEngineUtils/ExecutionEngineUtils.cpp:18-150 of the
// reference, except the median: the reference pivots at index n/2+1 (one past
// the middle, out of bounds for n <= 2); this one is the textbook median.
#ifndef IMEX_HIP_PROFILER_STATS_H
#define IMEX_HIP_PROFILER_STATS_H

#include <cstddef>
#include <vector>

namespace imexhip {

struct KernelTimeStats {
  float avg = 0, min = 0, max = 0, median = 0, stddev = 0, variance = 0, p95 = 0, p5 = 0,
        middleThirdAvg = 0;
};

KernelTimeStats computeStats(const std::vector<float> &timesMs);

} // namespace imexhip
#endif
