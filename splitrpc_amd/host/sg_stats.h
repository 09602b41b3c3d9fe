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

// Index of the p-quantile among N sorted samples: round(p * (N - 1)).
static inline size_t sg_quantile_index(double p, size_t n)
{
  return n ? (size_t)std::llround(p * (double)(n - 1)) : 0;
}

// The sample at that index of the sorted samples (0 for none).  The vector is left as it was.
static inline double getPercentile(const std::vector<uint64_t> &v, double p)
{
  const size_t k = sg_quantile_index(p, v.size());
  if (k >= v.size()) return 0.0;
  std::vector<uint64_t> sorted(v);
  std::sort(sorted.begin(), sorted.end());
  return (double)sorted[k];
}

static inline double getMean(const std::vector<uint64_t> &v)
{
  if (v.empty()) return 0.0;
  long double sum = 0.0L;
  for (uint64_t x : v) sum += (long double)x;
  return (double)(sum / (long double)v.size());
}

// The seven numbers of the summary line, in its order.
struct SgStatLine {
  double v[7];  // N, mean, p90, p95, p99, min, max
};

// One sort serves the three quantiles and both ends.
static inline SgStatLine sg_stat_line(std::vector<uint64_t> v)
{
  SgStatLine s{};
  s.v[0] = (double)v.size();
  if (v.empty()) return s;
  s.v[1] = getMean(v);
  std::sort(v.begin(), v.end());
  const double q[3] = {0.90, 0.95, 0.99};
  for (int i = 0; i < 3; i++) s.v[2 + i] = (double)v[sg_quantile_index(q[i], v.size())];
  s.v[5] = (double)v.front();
  s.v[6] = (double)v.back();
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
