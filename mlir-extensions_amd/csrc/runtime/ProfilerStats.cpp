#include "ProfilerStats.h"

#include <algorithm>
#include <cmath>
#include <limits>

namespace imexhip {

KernelTimeStats computeStats(const std::vector<float> &timesMs) {
  KernelTimeStats s;
  const size_t n = timesMs.size();
  if (n == 0) {
    // Same conventions as the reference for an empty run list.
    s.min = std::numeric_limits<float>::max();
    s.max = std::numeric_limits<float>::min();
    return s;
  }
  std::vector<float> sorted(timesMs);
  std::sort(sorted.begin(), sorted.end());
  s.min = sorted.front();
  s.max = sorted.back();

  // Mean: f32 running sum in run order, divided by n.
  float sum = 0.0f;
  for (float v : timesMs)
    sum += v;
  s.avg = sum / static_cast<float>(n);

  s.median = (n % 2) ? sorted[n / 2] : (sorted[n / 2] + sorted[n / 2 - 1]) / 2;

  // Population variance about the f32 mean, in run order.
  float sq = 0.0f;
  for (float v : timesMs)
    sq += (v - s.avg) * (v - s.avg);
  s.variance = sq / static_cast<float>(n);
  s.stddev = std::sqrt(s.variance);

  auto at = [&](double frac) {
    size_t idx = static_cast<size_t>(frac * static_cast<double>(n));
    if (idx >= n)
      idx = n - 1;
    return sorted[idx];
  };
  s.p95 = at(0.95);
  s.p5 = at(0.05);

  if (n < 3) {
    s.middleThirdAvg = s.median;
  } else {
    const size_t start = n / 3, end = n - start;
    float mid = 0.0f;
    for (size_t i = start; i < end; ++i)
      mid += sorted[i];
    s.middleThirdAvg = mid / static_cast<float>(end - start);
  }
  return s;
}

} // namespace imexhip
