// The host side of sampling: the random stream, and the pick from a position's candidates.
//
// Order of operations, as the reference's sampler (src/sample.rs:1-4, 179-190): repeat
// penalty -> top-k -> top-p -> min-p -> temperature -> one draw.  Penalty and top-k run on the
// device when k fits (csrc/sampling.hip) and hand over k 64-bit keys; otherwise the whole row
// comes here.  Everything after the candidates is float64, as in the reference
// (src/sample.rs:465-556).  Exactly one number is taken from the stream per decided token
// (src/sample.rs:272-277), so a seed gives the same tokens however requests are batched.
//
// `kept`, `draw` and `pick_sorted` below follow src/sample.rs:465-556 operation by operation, on
// purpose: the same tokens for the same seed need the same float64 operations in the same order,
// so here the reference's algorithm is the specification, not one choice among several.
#include <math.h>
#include <stdint.h>
#include <string.h>

#include <algorithm>
#include <functional>
#include <vector>

namespace {

uint64_t splitmix(uint64_t& s) {  // src/sample.rs:202-208
  s += 0x9e3779b97f4a7c15ull;
  uint64_t z = s;
  z = (z ^ (z >> 30)) * 0xbf58476d1ce4e5b9ull;
  z = (z ^ (z >> 27)) * 0x94d049bb133111ebull;
  return z ^ (z >> 31);
}

inline uint64_t rotl(uint64_t x, int k) { return (x << k) | (x >> (64 - k)); }

// The order key of a logit (src/sample.rs:280-293): larger logit, larger key; -0.0 ties +0.0;
// NaN below everything.
uint32_t order_key(float v) {
  if (v != v) return 0;
  uint32_t b;
  memcpy(&b, &v, 4);
  if (v == 0.0f) b = 0;
  return (b >> 31) ? ~b : (b | 0x80000000u);
}

float unkey(uint32_t k) {
  uint32_t b = (k >> 31) ? (k & 0x7fffffffu) : ~k;
  float v;
  memcpy(&v, &b, 4);
  return v;
}

// How many candidates (best first) survive top-p then min-p: at least one
// (src/sample.rs:465-500).
int kept(const std::vector<float>& logit, float top_p, float min_p) {
  int n = 0;
  while (n < (int)logit.size() && logit[n] == logit[n]) ++n;
  const double l0 = logit[0];
  if (n <= 1 || !std::isfinite(l0)) return 1;
  if (top_p < 1.0f) {
    std::vector<double> e(n);
    double z = 0.0;
    for (int i = 0; i < n; ++i) {
      e[i] = exp((double)logit[i] - l0);
      z += e[i];
    }
    double cum = 0.0;
    int cut = n;
    for (int i = 0; i < n; ++i) {
      cum += e[i] / z;
      if (cum >= (double)top_p) {
        cut = i + 1;
        break;
      }
    }
    n = cut;
  }
  if (min_p > 0.0f) {
    const double lo = l0 + log((double)min_p);
    int m = 0;
    while (m < n && (double)logit[m] >= lo) ++m;
    n = std::max(m, 1);
  }
  return n;
}

// The inverse CDF (src/sample.rs:542-556): the first i whose cumulative weight passes u * total;
// the target stays below the total; never a zero-weight index.
int draw(const std::vector<double>& w, double u) {
  double z = 0.0;
  for (double x : w) z += x;
  const double target = std::min(u * z, nextafter(z, -INFINITY));
  double cum = 0.0;
  int last = 0;
  for (int i = 0; i < (int)w.size(); ++i) {
    if (w[i] > 0.0) last = i;
    cum += w[i];
    if (target < cum) return i;
  }
  return last;
}

int pick_sorted(const std::vector<uint64_t>& keys, float temp, float top_p, float min_p, double u) {
  std::vector<float> logit(keys.size());
  for (size_t i = 0; i < keys.size(); ++i) logit[i] = unkey((uint32_t)(keys[i] >> 32));
  const int n = kept(logit, top_p, min_p);
  if (n == 1) return (int)(uint32_t)keys[0];
  const double l0 = logit[0], t = temp;
  std::vector<double> w(n);
  for (int i = 0; i < n; ++i) w[i] = exp(((double)logit[i] - l0) / t);
  return (int)(uint32_t)keys[draw(w, u)];
}

}  // namespace

extern "C" {

// xoshiro256** seeded by four splitmix64 outputs (src/sample.rs:212-242).
void axh_rng_seed(uint64_t seed, uint64_t state[4]) {
  uint64_t s = seed;
  for (int i = 0; i < 4; ++i) state[i] = splitmix(s);
}

uint64_t axh_rng_next_u64(uint64_t s[4]) {
  const uint64_t r = rotl(s[1] * 5, 7) * 9;
  const uint64_t t = s[1] << 17;
  s[2] ^= s[0];
  s[3] ^= s[1];
  s[1] ^= s[2];
  s[0] ^= s[3];
  s[2] ^= t;
  s[3] = rotl(s[3], 45);
  return r;
}

// Uniform in [0, 1), 53 bits.
double axh_rng_next_f64(uint64_t s[4]) { return (double)(axh_rng_next_u64(s) >> 11) * (1.0 / 9007199254740992.0); }

// The pick from k candidate keys in any order (the device's top-k output).
int axh_sample_pick_keys(const uint64_t* keys, int k, float temp, float top_p, float min_p, double u) {
  if (k <= 0) return -1;
  std::vector<uint64_t> sorted(keys, keys + k);
  std::sort(sorted.begin(), sorted.end(), std::greater<uint64_t>());
  return pick_sorted(sorted, temp, top_p, min_p, u);
}

// The picks of a step's rows in one call: row r has k[r] candidate keys at keys + r * k_stride and
// takes one number from its own stream states[r] (four 64-bit words), as one
// axh_sample_pick_keys(.., axh_rng_next_f64(states[r])) per row would.
void axh_sample_pick_keys_rows(const uint64_t* keys, int k_stride, int n_rows, const int* k, const float* temp,
                               const float* top_p, const float* min_p, uint64_t* const* states, int* picks) {
  for (int r = 0; r < n_rows; ++r)
    picks[r] = axh_sample_pick_keys(keys + (size_t)r * k_stride, k[r], temp[r], top_p[r], min_p[r],
                                    axh_rng_next_f64(states[r]));
}

// The whole pipeline on a row of logits held by the host (top_k 0: every token is a
// candidate).  `recent`: the ids the penalty looks at (already cut to the last N); the
// penalty divides a positive logit and multiplies any other (src/sample.rs:307-326).
int axh_sample_pick_row(const float* logits, int n, const int* recent, int n_recent, float penalty, int top_k,
                        float temp, float top_p, float min_p, double u) {
  if (n <= 0) return -1;
  std::vector<float> l(logits, logits + n);
  if (penalty != 1.0f && n_recent > 0) {
    std::vector<int> ids(recent, recent + n_recent);
    std::sort(ids.begin(), ids.end());
    ids.erase(std::unique(ids.begin(), ids.end()), ids.end());
    for (int id : ids)
      if (id >= 0 && id < n) l[id] = l[id] > 0.0f ? l[id] / penalty : l[id] * penalty;
  }
  std::vector<uint64_t> keys(n);
  for (int i = 0; i < n; ++i) keys[i] = ((uint64_t)order_key(l[i]) << 32) | (uint32_t)i;
  const int k = top_k <= 0 || top_k > n ? n : top_k;
  std::partial_sort(keys.begin(), keys.begin() + k, keys.end(), std::greater<uint64_t>());
  keys.resize(k);
  return pick_sorted(keys, temp, top_p, min_p, u);
}

// The greedy pick of a host row: the largest key (ties to the last index, NaN never).
int axh_argmax_row(const float* logits, int n) {
  uint64_t best = 0;
  for (int i = 0; i < n; ++i) best = std::max(best, ((uint64_t)order_key(logits[i]) << 32) | (uint32_t)i);
  return (int)(uint32_t)best;
}

}  // extern "C"
