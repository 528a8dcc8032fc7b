// Could the column sums of sum_rows (signed terms) be built from runs the way the softmax row
// sum is? While the running sum S of a left-to-right float sum stays in one binade and keeps
// its sign, every step fl(S + t) equals S + rne(t / ulp) * ulp (ties aside): integer adds, so a
// run of such steps is ONE addend. This program measures the best any plan of that kind can do
// on the benchmark's columns - 16384 terms drawn N(0, 1) - by cutting each column into runs
// with full knowledge of the true running sums, at several granularities (a block of g terms
// is either wholly inside one run or handed to the chain term by term), rebuilding the sum
// from the runs and checking it bit for bit against the serial loop. It prints, per
// granularity, the share of a column's 16384 dependent adds that is left for the chain.
#include <cmath>
#include <cstdint>
#include <cstdio>
#include <cstring>
#include <random>
#include <vector>

static uint32_t Bits(float f) {
  uint32_t u;
  std::memcpy(&u, &f, 4);
  return u;
}
static int Binade(float s) { return static_cast<int>((Bits(s) >> 23) & 0xff); }  // 0 for zero / subnormal
static bool Negative(float s) { return (Bits(s) >> 31) != 0; }

// One step inside a run: S and the result are normal, same sign, same binade, and t is no tie
// on that binade's grid. Then fl(S + t) - S is the multiple of ulp nearest t.
static bool StepStaysInRun(float s, float t, float r) {
  if (Binade(s) == 0 || Binade(s) == 255 || Binade(r) != Binade(s) || Negative(r) != Negative(s)) return false;
  const double ulp = std::ldexp(1.0, Binade(s) - 127 - 23);
  const double q = static_cast<double>(t) / ulp;
  const double frac = q - std::floor(q);
  return frac != 0.5;
}

int main(int argc, char **argv) {
  const int rows = 16384;
  const int columns = argc > 1 ? std::atoi(argv[1]) : 256;
  std::mt19937 gen(6);
  std::normal_distribution<float> normal(0.0f, 1.0f);
  const int grains[] = {1, 4, 16, 64, 256};
  double left[5] = {0, 0, 0, 0, 0};
  std::vector<float> t(rows), s(rows + 1);
  std::vector<char> clean(rows);
  for (int c = 0; c < columns; ++c) {
    for (int y = 0; y < rows; ++y) t[y] = normal(gen);
    // the reference's loop (tensor_cpu-inl.h:221-227): res = src(0, x); res += src(y, x)
    volatile float acc = t[0];
    s[0] = 0.0f;
    s[1] = acc;
    clean[0] = 0;
    for (int y = 1; y < rows; ++y) {
      const float before = acc;
      acc = acc + t[y];
      s[y + 1] = acc;
      clean[y] = StepStaysInRun(before, t[y], acc) ? 1 : 0;
    }
    for (int gi = 0; gi < 5; ++gi) {
      const int g = grains[gi];
      // a block is clean if every step in it stays in the run that the step before the
      // block was in (first step included: it continues the run)
      size_t addends = 0;
      bool in_run = false;
      int run_binade = -1;
      // rebuild the sum from the plan and compare
      float sum = 0.0f;
      int64_t run_q = 0;
      double run_ulp = 0.0;
      auto close_run = [&]() {
        if (in_run) {
          sum = static_cast<float>(static_cast<double>(sum) + static_cast<double>(run_q) * run_ulp);
          in_run = false;
        }
      };
      for (int b = 0; b < rows; b += g) {
        bool ok = true;
        for (int y = b; y < b + g && y < rows; ++y) ok = ok && clean[y];
        if (ok && in_run && Binade(s[b]) != run_binade) ok = false;
        if (ok) {
          if (!in_run) {
            in_run = true;
            run_binade = Binade(s[b]);
            run_q = 0;
            run_ulp = std::ldexp(1.0, run_binade - 127 - 23);
            ++addends;
          }
          for (int y = b; y < b + g && y < rows; ++y) {
            run_q += static_cast<int64_t>(std::nearbyint(static_cast<double>(t[y]) / run_ulp));
          }
        } else {
          close_run();
          for (int y = b; y < b + g && y < rows; ++y) {
            volatile float v = sum;
            v = v + t[y];
            sum = v;
            ++addends;
          }
        }
      }
      close_run();
      if (Bits(sum) != Bits(s[rows])) {
        std::printf("MISMATCH column %d grain %d: %a vs %a\n", c, g, sum, s[rows]);
        return 1;
      }
      left[gi] += static_cast<double>(addends) / rows;
    }
  }
  std::printf("OK %d columns of %d terms; share of the dependent adds left for the chain:", columns, rows);
  for (int gi = 0; gi < 5; ++gi) std::printf(" grain %d: %.3f", grains[gi], left[gi] / columns);
  std::printf("\n");
  return 0;
}
