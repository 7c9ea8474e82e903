// extern "C" entry points over the reference's own profiler statistics
// (lib/ExecutionEngine/ExecutionEngineUtils/ExecutionEngineUtils.cpp, compiled
// from the reference checkout by the Makefile beside this file).  TEST
// INFRASTRUCTURE ONLY: used to validate the oracle's restatement of them.
#include "imex/ExecutionEngine/ExecutionEngineUtils.h"

#include <cstddef>
#include <vector>

namespace {
std::vector<float> vec(const float *v, size_t n) { return std::vector<float>(v, v + n); }
} // namespace

extern "C" {
float ref_stat_min(const float *v, size_t n) { return calculateMin(vec(v, n)); }
float ref_stat_max(const float *v, size_t n) { return calculateMax(vec(v, n)); }
float ref_stat_avg(const float *v, size_t n) { return calculateAverage(vec(v, n)); }
float ref_stat_median(const float *v, size_t n) {
  auto x = vec(v, n);
  return calculateMedian(x);
}
float ref_stat_stddev(const float *v, size_t n) { return calculateStdDev(vec(v, n)); }
float ref_stat_variance(const float *v, size_t n) { return calculateVariance(vec(v, n)); }
float ref_stat_p95(const float *v, size_t n) {
  auto x = vec(v, n);
  return calculateP95(x);
}
float ref_stat_p5(const float *v, size_t n) {
  auto x = vec(v, n);
  return calculateP5(x);
}
float ref_stat_middle_third_avg(const float *v, size_t n) {
  auto x = vec(v, n);
  return calculateMiddleThirdAverage(x);
}
}
