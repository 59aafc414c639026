// Random numbers for weight initialisation and dataset shuffling.  The
// reference seeds a Mersenne twister from the clock (Rng.cpp:7-16); this one
// can also be given a seed so that a run is repeatable.
#pragma once
#include <random>
#include <vector>

class RNG {
public:
  std::mt19937 gen;
  RNG();
  explicit RNG(unsigned seed);
  int randint(int n);
  float uniform(float a = 0, float b = 1);
  float normal(float mean = 0, float sd = 1);
  int bernoulli(float p);
  template <typename T> void vectorShuffle(std::vector<T> &v) {
    for (int i = (int)v.size() - 1; i > 0; --i)
      std::swap(v[i], v[randint(i + 1)]);
  }
  // m of the numbers 0..n-1, ascending (all of them when m == n)
  std::vector<int> NchooseM(int n, int m);
};
