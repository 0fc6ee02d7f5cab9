#include "Rand.h"

#include <cmath>
#include <stdexcept>
#include <unordered_map>

namespace {

constexpr std::uint64_t kGolden = 0x9E3779B97F4A7C15ull;

inline std::uint64_t mix64(std::uint64_t z) {
  z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
  z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
  return z ^ (z >> 31);
}

struct StreamState {
  std::uint64_t seed = 0;
  std::uint64_t stream = 0;
  std::uint64_t key = mix64(kGolden);  // mix64(seed + GOLDEN*(stream+1))
  std::uint64_t counter = 0;
  void rekey() { key = mix64(seed + kGolden * (stream + 1)); }
  std::uint64_t next() { return mix64(key + kGolden * (++counter)); }
};

StreamState g_state;

inline double unit24(std::uint64_t raw) { return (double)(raw >> 40) * 0x1p-24; }

template <typename T>
void fill_uniform(T* out, std::size_t len, T low, T high) {
  const T span = high - low;
  for (std::size_t i = 0; i < len; ++i) out[i] = low + span * (T)unit24(g_state.next());
}

template <typename T>
void fill_ints(T* out, int len, int low, int high, bool duplicates) {
  if (len <= 0) return;
  const std::uint64_t span = (std::uint64_t)((std::int64_t)high - low) + 1;
  if (duplicates) {
    for (int i = 0; i < len; ++i) out[i] = (T)(low + (std::int64_t)(g_state.next() % span));
    return;
  }
  if ((std::uint64_t)len > span) throw std::invalid_argument("randFill: range smaller than len");
  // Partial Fisher-Yates over the virtual array [0, span): `moved` records only the slots that
  // no longer hold their own index, so memory stays O(len).
  std::unordered_map<std::uint64_t, std::uint64_t> moved;
  auto at = [&](std::uint64_t k) {
    auto it = moved.find(k);
    return it == moved.end() ? k : it->second;
  };
  for (int i = 0; i < len; ++i) {
    std::uint64_t j = (std::uint64_t)i + g_state.next() % (span - (std::uint64_t)i);
    std::uint64_t vi = at((std::uint64_t)i), vj = at(j);
    out[i] = (T)(low + (std::int64_t)vj);
    moved[j] = vi;
  }
}

}  // namespace

void randSeed(std::uint64_t seed) {
  g_state.seed = seed;
  g_state.stream = 0;
  g_state.counter = 0;
  g_state.rekey();
}

void randStream(std::uint64_t stream) {
  g_state.stream = stream;
  g_state.counter = 0;
  g_state.rekey();
}

std::uint64_t randRaw(std::uint64_t seed, std::uint64_t stream, std::uint64_t counter) {
  return mix64(mix64(seed + kGolden * (stream + 1)) + kGolden * (counter + 1));
}

void randFill(float* array, std::size_t len, const float low, const float high, bool) {
  fill_uniform<float>(array, len, low, high);
}

void randFill(double* array, std::size_t len, const double low, const double high, bool) {
  fill_uniform<double>(array, len, low, high);
}

void randFill(aligned_vector<float>& vec, const float low, const float high) {
  fill_uniform<float>(vec.data(), vec.size(), low, high);
}

void randFill(aligned_vector<double>& vec, const double low, const double high) {
  fill_uniform<double>(vec.data(), vec.size(), low, high);
}

void randFill(int* array, int len, const int low, const int high, bool duplicates) {
  fill_ints<int>(array, len, low, high, duplicates);
}

void randFill(std::int64_t* array, int len, const int low, const int high, bool duplicates) {
  fill_ints<std::int64_t>(array, len, low, high, duplicates);
}

void randFill(aligned_vector<int>& vec, const int low, const int high, bool duplicates) {
  fill_ints<int>(vec.data(), (int)vec.size(), low, high, duplicates);
}

void randFill(aligned_vector<std::int64_t>& vec, const int low, const int high, bool duplicates) {
  fill_ints<std::int64_t>(vec.data(), (int)vec.size(), low, high, duplicates);
}

void randFillNormal(float* array, std::size_t len, const float mean, const float stddev) {
  constexpr double kTwoPi = 6.283185307179586476925286766559;
  for (std::size_t i = 0; i < len; ++i) {
    double u1 = ((double)(g_state.next() >> 40) + 1.0) * 0x1p-24;  // (0, 1]
    double u2 = unit24(g_state.next());                            // [0, 1)
    double z = std::sqrt(-2.0 * std::log(u1)) * std::cos(kTwoPi * u2);
    array[i] = mean + stddev * (float)z;
  }
}
