// Seeded random weights whose every value is a function of (seed, tensor index, element index)
// alone, so that any number of threads, and any other implementation of the same few lines,
// gives the same bits.  (The reference's tests draw their weights from an empty VarMap, whose
// distribution its text does not state: crates/engine/src/testing.rs:68-77.)
//
//   mix(x):   x += 0x9E3779B97F4A7C15; x = (x ^ x >> 30) * 0xBF58476D1CE4E5B9;
//             x = (x ^ x >> 27) * 0x94D049BB133111EB; return x ^ x >> 31      (splitmix64)
//   key     = mix(seed ^ mix(tensor))
//   pair j  : a = mix(key + 2 j), b = mix(key + 2 j + 1)
//             u1 = ((a >> 11) + 0.5) / 2^53,  u2 = ((b >> 11) + 0.5) / 2^53   (both in (0, 1))
//             r = sqrt(-2 ln u1);  z[2 j] = r cos(2 pi u2);  z[2 j + 1] = r sin(2 pi u2)
//   value i = (float)(mean + std * z[i])                  (Box-Muller, double until the end)
#include <cmath>
#include <cstdint>
#include <thread>
#include <vector>

#define RT_API extern "C" __attribute__((visibility("default")))

namespace {

inline uint64_t mix(uint64_t x) {
  x += 0x9E3779B97F4A7C15ull;
  x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
  x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
  return x ^ (x >> 31);
}

void fill_pairs(float* out, long long n, uint64_t key, double mean, double std_dev,
                long long first_pair, long long last_pair) {
  const double two_pi = 6.283185307179586476925286766559;
  const double scale = 1.0 / 9007199254740992.0;   // 2^-53
  for (long long j = first_pair; j < last_pair; ++j) {
    const uint64_t a = mix(key + 2 * (uint64_t)j), b = mix(key + 2 * (uint64_t)j + 1);
    const double u1 = ((double)(a >> 11) + 0.5) * scale;
    const double u2 = ((double)(b >> 11) + 0.5) * scale;
    const double r = std::sqrt(-2.0 * std::log(u1));
    const double angle = two_pi * u2;
    out[2 * j] = (float)(mean + std_dev * (r * std::cos(angle)));
    if (2 * j + 1 < n) out[2 * j + 1] = (float)(mean + std_dev * (r * std::sin(angle)));
  }
}

}  // namespace

// out[0 .. n) = mean + std * N(0, 1), float32, from (seed, tensor); `threads` workers
// (0: as many as the machine has) split the pairs, which changes nothing of the result.
RT_API int rlis_fill_normal(float* out, long long n, unsigned long long seed,
                            unsigned long long tensor, double mean, double std_dev, int threads) {
  if (n < 0 || !out) return -1;
  const uint64_t key = mix(seed ^ mix(tensor));
  const long long pairs = (n + 1) / 2;
  int workers = threads > 0 ? threads : (int)std::thread::hardware_concurrency();
  if (workers < 1) workers = 1;
  if (pairs < 1 << 16) workers = 1;
  if (workers == 1) {
    fill_pairs(out, n, key, mean, std_dev, 0, pairs);
    return 0;
  }
  std::vector<std::thread> pool;
  const long long per = (pairs + workers - 1) / workers;
  for (int w = 0; w < workers; ++w) {
    const long long lo = w * per, hi = lo + per < pairs ? lo + per : pairs;
    if (lo >= hi) break;
    pool.emplace_back(fill_pairs, out, n, key, mean, std_dev, lo, hi);
  }
  for (auto& t : pool) t.join();
  return 0;
}
