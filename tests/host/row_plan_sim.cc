// Host model of the planned row sum of the softmax kernel (mshadow_amd/csrc/softmax_kernels.h,
// RowOrderedSum): the row is cut into chunks of 64 lanes x N terms, the chunks and lanes are
// classified from approximate prefix sums with the very functions the device code uses
// (mshadow_amd/csrc/ordered_sum.h), the list of addends is built and summed serially, and every
// run is verified on the sums obtained. The result must equal a plain serial float loop bit
// for bit on every row, whether the plan held or the fall-back was taken; rows shaped like a
// softmax's must not need the fall-back. Prints "OK <cases> <fallbacks>" and exits 0.
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstdlib>
#include <random>
#include <vector>

#include "../../mshadow_amd/csrc/ordered_sum.h"

using namespace ordered_sum;

static float Serial(const std::vector<float> &t) {
  volatile float s = 0.0f;
  for (float v : t) s = s + v;
  return s;
}

struct Addend {
  float value;
  int check;  // binade the sum must be in before and after this addend; -1: a term, no check
};

template <int N>
static bool PlannedSum(const std::vector<float> &row, int max_slots, float *result, size_t *addends) {
  const int chunk_terms = 64 * N;
  std::vector<float> t(row);
  while (t.size() % chunk_terms) t.push_back(0.0f);
  const int nch = static_cast<int>(t.size() / chunk_terms);
  // A: approximate sum and largest term of every chunk
  std::vector<float> approx(nch), cmax(nch);
  for (int k = 0; k < nch; ++k) {
    float s = 0.0f, m = 0.0f;
    for (int l = 0; l < 64; ++l) {
      float a = 0.0f;
      for (int i = 0; i < N; ++i) {
        const float v = t[(k * 64 + l) * N + i];
        a += v;
        m = (m < v) ? v : m;
      }
      s += a;
    }
    approx[k] = s;
    cmax[k] = m;
  }
  // B: plan per chunk
  std::vector<float> start(nch), lowb(nch);
  std::vector<int> code(nch);
  {
    float pre = 0.0f, seen_max = 0.0f;
    int prev = -1;
    for (int k = 0; k < nch; ++k) {
      start[k] = pre;
      const float low = std::fmax(PlanLowBound(pre, static_cast<float>(k) * chunk_terms), seen_max);
      lowb[k] = low;
      pre += approx[k];
      seen_max = std::fmax(seen_max, cmax[k]);
      int c = PlanBinade(low, PlanHighBound(pre));
      if (c >= 0 && prev >= 0 && prev != c) c = -1;  // a run has one binade
      code[k] = c;
      prev = c;
    }
    if (pre != pre) {  // NaN among the terms
      *result = pre;
      return true;
    }
  }
  // C: integer totals of the clean chunks, addend lists of the others
  std::vector<Addend> list;
  uint32_t run = 0;
  int run_e = -1;
  int slots = 0;
  auto flush = [&]() {
    if (run_e >= 0) list.push_back({RunAddend(static_cast<uint32_t>(run_e), run), run_e});
    run = 0;
    run_e = -1;
  };
  for (int k = 0; k < nch; ++k) {
    const float(*lane)[N] = reinterpret_cast<const float(*)[N]>(&t[static_cast<size_t>(k) * chunk_terms]);
    bool whole = code[k] >= 0;
    uint32_t total = 0;
    if (whole) {
      for (int l = 0; l < 64; ++l) {
        const LaneQuantum q = LaneDualQuant<N>(lane[l], static_cast<uint32_t>(code[k]));
        whole = whole && q.ok;
        total += q.q;
      }
    }
    if (whole) {
      total = total < (1u << 24) ? total : (1u << 24);
      run += total;
      run_e = code[k];
      continue;
    }
    flush();
    if (++slots > max_slots) return false;
    // lane-level plan of a chunk that is not clean as a whole
    float incl = 0.0f, seen = 0.0f;
    int prev = -1;
    uint32_t lrun = 0;
    for (int l = 0; l < 64; ++l) {
      float a = 0.0f, m = 0.0f;
      for (int i = 0; i < N; ++i) {
        a += lane[l][i];
        m = (m < lane[l][i]) ? lane[l][i] : m;
      }
      const float before = start[k] + incl;
      incl += a;
      const float after = start[k] + incl;
      float low = PlanLowBound(before, static_cast<float>((k * 64 + l) * N));
      low = std::fmax(std::fmax(low, seen), lowb[k]);
      seen = std::fmax(seen, m);
      int c = PlanBinade(low, PlanHighBound(after));
      LaneQuantum q = {0u, false};
      if (c >= 0) q = LaneDualQuant<N>(lane[l], static_cast<uint32_t>(c));
      if (!q.ok) c = -1;
      if (c < 0 || c != prev) {
        if (prev >= 0) list.push_back({RunAddend(static_cast<uint32_t>(prev), lrun), prev});
        lrun = 0;
      }
      if (c < 0) {
        for (int i = 0; i < N; ++i) list.push_back({lane[l][i], -1});
      } else {
        lrun += q.q;
      }
      prev = c;
    }
    if (prev >= 0) list.push_back({RunAddend(static_cast<uint32_t>(prev), lrun), prev});
  }
  flush();
  // the chain, with the verification of every run
  float s = 0.0f;
  for (const Addend &a : list) {
    const float before = s;
    s = s + a.value;
    if (a.check >= 0 && !RunHolds(before, s, static_cast<uint32_t>(a.check))) return false;
  }
  *result = s;
  *addends += list.size();
  return true;
}

static long g_cases = 0, g_fallbacks = 0;
static size_t g_addends = 0;

template <int N>
static bool Check(const std::vector<float> &row, const char *name, bool must_hold) {
  float got = 0.0f;
  bool negative = false;
  for (float v : row) negative = negative || v < 0.0f;
  const bool held = !negative && PlannedSum<N>(row, 24, &got, &g_addends);
  const float want = Serial(row);
  ++g_cases;
  if (!held) {
    ++g_fallbacks;
    if (must_hold) {
      fprintf(stderr, "PLAN DID NOT HOLD %s N=%d n=%zu\n", name, N, row.size());
      return false;
    }
    return true;  // the device code then sums the row by wave scans
  }
  if (BitsOf(got) != BitsOf(want) && !(std::isnan(got) && std::isnan(want))) {
    fprintf(stderr, "MISMATCH %s N=%d n=%zu got %a want %a\n", name, N, row.size(), got, want);
    return false;
  }
  return true;
}

static bool CheckAll(const std::vector<float> &row, const char *name, bool must_hold = false) {
  return Check<4>(row, name, must_hold) && Check<1>(row, name, false) && Check<2>(row, name, false);
}

int main() {
  std::mt19937 rng(4321);
  std::normal_distribution<float> normal(0.0f, 1.0f);
  std::uniform_real_distribution<float> uni(0.0f, 1.0f);
  bool ok = true;
  // 1. softmax-like rows: exp(x - max), x ~ N(0, sigma); the plan must hold for these
  for (float sigma : {0.1f, 1.0f, 3.0f, 6.0f}) {
    for (int n : {257, 1000, 4096, 32000, 65536}) {
      for (int rep = 0; rep < 12; ++rep) {
        std::vector<float> x(n);
        float mx = -INFINITY;
        for (auto &v : x) { v = normal(rng) * sigma; mx = std::fmax(mx, v); }
        for (auto &v : x) v = expf(v - mx);
        ok = CheckAll(x, "softmax", true) && ok;
      }
    }
  }
  // one class far above the others (the sum sits just above 1 from there on), at any position
  for (int rep = 0; rep < 40; ++rep) {
    const int n = 32000;
    std::vector<float> x(n);
    for (auto &v : x) v = normal(rng);
    x[rng() % n] += 10.0f + 30.0f * uni(rng);
    float mx = -INFINITY;
    for (auto v : x) mx = std::fmax(mx, v);
    for (auto &v : x) v = expf(v - mx);
    ok = CheckAll(x, "confident", true) && ok;
  }
  for (float sigma : {10.0f, 40.0f}) {
    for (int n : {1, 3, 64, 257, 1000, 4096, 32000}) {
      for (int rep = 0; rep < 6; ++rep) {
        std::vector<float> x(n);
        float mx = -INFINITY;
        for (auto &v : x) { v = normal(rng) * sigma; mx = std::fmax(mx, v); }
        for (auto &v : x) v = expf(v - mx);
        ok = CheckAll(x, "softmax-wide") && ok;
      }
    }
  }
  // 2. grids that produce exact ties
  for (int rep = 0; rep < 300; ++rep) {
    int n = 1 + rng() % 3000;
    std::vector<float> x(n);
    for (auto &v : x) v = std::ldexp(static_cast<float>(rng() % 64), -static_cast<int>(rng() % 30));
    ok = CheckAll(x, "ties") && ok;
  }
  for (int rep = 0; rep < 100; ++rep) {  // multiples of 1/8 and of 2^-24 next to a large first term
    int n = 1000 + rng() % 30000;
    std::vector<float> x(n);
    for (auto &v : x) v = std::ldexp(static_cast<float>(1 + rng() % 8), -3);
    ok = CheckAll(x, "eighths") && ok;
    for (auto &v : x) v = std::ldexp(static_cast<float>(rng() % 3), -24);
    x[0] += 1.0f;
    ok = CheckAll(x, "half-ulps") && ok;
  }
  // 3. constants
  for (float c : {1.0f, 0.5f, 3.0f, 1e-3f, 0.1f}) {
    std::vector<float> x(40000, c);
    ok = CheckAll(x, "const") && ok;
  }
  // 4. leading zeros / subnormals / tiny then large; ascending, descending, shuffled
  for (int rep = 0; rep < 90; ++rep) {
    int n = 500 + rng() % 5000;
    std::vector<float> x(n);
    for (int i = 0; i < n; ++i) {
      float e = -140.0f + 150.0f * i / n;
      x[i] = std::ldexp(1.0f + uni(rng), static_cast<int>(e));
      if (rng() % 7 == 0) x[i] = 0.0f;
    }
    if (rep % 3 == 1) std::reverse(x.begin(), x.end());
    if (rep % 3 == 2) std::shuffle(x.begin(), x.end(), rng);
    ok = CheckAll(x, "range") && ok;
  }
  {
    std::vector<float> x(3000, 0.0f);
    ok = CheckAll(x, "zeros", true) && ok;
    x[2999] = 1e-40f;
    ok = CheckAll(x, "zeros+denorm") && ok;
    x[10] = 3e-42f;
    ok = CheckAll(x, "denorms") && ok;
    x.assign(3000, 2.0e-39f);
    ok = CheckAll(x, "all denormal") && ok;
    x[1500] = INFINITY;
    ok = CheckAll(x, "inf") && ok;
    x[100] = NAN;
    ok = CheckAll(x, "nan") && ok;
    x.assign(5000, 3.0e38f);
    ok = CheckAll(x, "overflow") && ok;
    x.assign(5000, 0.25f);
    x[77] = -0.5f;
    ok = CheckAll(x, "negative") && ok;
  }
  // 5. uniform magnitudes, rare large terms, sums ending next to a power of two
  for (int rep = 0; rep < 60; ++rep) {
    int n = 20000 + rng() % 20000;
    std::vector<float> x(n);
    for (auto &v : x) v = uni(rng);
    ok = CheckAll(x, "uniform", true) && ok;
    for (int i = 0; i < n; ++i) x[i] = (i % 97 == 0) ? 1.0f : 1e-7f;
    ok = CheckAll(x, "rare large") && ok;
    for (auto &v : x) v = std::ldexp(1.0f, static_cast<int>(rng() % 60) - 40);
    ok = CheckAll(x, "dynamic range") && ok;
  }
  if (!ok) return 1;
  printf("OK %ld cases, %ld fall-backs, %.1f addends per planned row\n", g_cases, g_fallbacks,
         static_cast<double>(g_addends) / (g_cases - g_fallbacks));
  return 0;
}
