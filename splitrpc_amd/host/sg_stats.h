// sg_stats.h -- nanosecond samples and their one-line summary, as the reference
// keeps and prints them under PROFILE_MODE: getCurNs (src/utils/time_utils.h:49-55),
// getPercentile / getMean / print_stat (src/utils/stats_utils.h:10-31,69-79),
// PROF_PRINT (src/utils/time_utils.h:27-38).  Same names, same output line:
//   <key> stats(ns) [N, Mean, p90, p95, p99, min, max]: ...
#pragma once

#include <time.h>

#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <string>
#include <vector>

static inline uint64_t getCurNs()
{
  struct timespec ts;
  clock_gettime(CLOCK_MONOTONIC, &ts);
  return (uint64_t)ts.tv_sec * 1000000000ull + (uint64_t)ts.tv_nsec;
}

// The sample at index round(p * (N - 1)) of the sorted samples (0 for none).
static inline double getPercentile(std::vector<uint64_t> &v, double p)
{
  if (v.empty()) return 0.0;
  const size_t k = (size_t)std::llround(p * (double)(v.size() - 1));
  if (k >= v.size()) return 0.0;
  std::nth_element(v.begin(), v.begin() + k, v.end());
  return (double)v[k];
}

static inline double getMean(const std::vector<uint64_t> &v)
{
  double mean = 0.0;
  uint64_t n = 0;
  for (uint64_t x : v) mean += ((double)x - mean) / (double)++n;
  return mean;
}

// The seven numbers of the summary line, in its order.
struct SgStatLine {
  double v[7];  // N, mean, p90, p95, p99, min, max
};

static inline SgStatLine sg_stat_line(std::vector<uint64_t> v)
{
  SgStatLine s{};
  s.v[0] = (double)v.size();
  if (v.empty()) return s;
  s.v[1] = getMean(v);
  s.v[2] = getPercentile(v, 0.90);
  s.v[3] = getPercentile(v, 0.95);
  s.v[4] = getPercentile(v, 0.99);
  s.v[5] = (double)*std::min_element(v.begin(), v.end());
  s.v[6] = (double)*std::max_element(v.begin(), v.end());
  return s;
}

static inline void print_stat(const std::string &key, const std::vector<uint64_t> &vec)
{
  const SgStatLine s = sg_stat_line(vec);
  std::printf("%s stats(ns) [N, Mean, p90, p95, p99, min, max]: %zu, %0.2f, %0.2f, %0.2f, %0.2f, %llu, %llu\n",
              key.c_str(), vec.size(), s.v[1], s.v[2], s.v[3], s.v[4], (unsigned long long)s.v[5],
              (unsigned long long)s.v[6]);
}

#ifdef PROFILE_MODE
#define PROF_PRINT(key, vec) \
  do {                       \
    if (!(vec).empty()) print_stat(key, vec); /* an engine that made no such call prints no line */ \
  } while (0)
#else
#define PROF_PRINT(key, vec)
#endif
