// A second plain implementation of the dense Llama decoder, independent of the first
// (plain_llama.py) and of the engine: scalar loops over whole sequences on the host, float32
// values with float64 accumulators for every sum, a contiguous key/value array per sequence,
// no cache reuse, no library.  Written from the reference's formulas, read, not run; every
// function cites the lines under /root/reference/ it follows.  The tests compile it with g++
// and compare it with the torch twin and with the engine.
#include <cmath>
#include <cstdint>
#include <vector>

extern "C" {

struct PlainConfig {
  int hidden, intermediate, layers, heads, kv_heads, head_dim, vocab;
  int tied;                       // lm_head is the embedding table (llama.rs:152-156)
  float eps, theta;
  int scaled;                     // rope_scaling of type llama3 present
  float factor, low_freq_factor, high_freq_factor, original_max_positions;
};

struct PlainLayer {
  const float *input_norm, *q, *k, *v, *o, *post_norm, *gate, *up, *down;
};

}  // extern "C"

namespace {

// y = x / sqrt(mean(x^2) + eps) * w; the weight multiplies directly, it is not 1 + w
// (crates/model/src/layers.rs:112-118, 141-146).
void rms_norm(const float* x, const float* w, float eps, int n, float* y) {
  double ss = 0.0;
  for (int i = 0; i < n; ++i) ss += (double)x[i] * x[i];
  const float inv = 1.0f / std::sqrt((float)(ss / n) + eps);
  for (int i = 0; i < n; ++i) y[i] = x[i] * inv * w[i];
}

// y[o] = sum_i x[i] W[o][i]: bias-free, W stored (out, in) (layers.rs:17-19, 72-99).
void linear(const float* x, const float* w, int in, int out, float* y) {
  for (int o = 0; o < out; ++o) {
    double s = 0.0;
    const float* row = w + (long long)o * in;
    for (int i = 0; i < in; ++i) s += (double)x[i] * row[i];
    y[o] = (float)s;
  }
}

// Inverse frequencies in float32, with the three bands of llama3 scaling
// (crates/model/src/rope.rs:19-49).
std::vector<float> inverse_frequencies(const PlainConfig& c) {
  std::vector<float> f;
  for (int i = 0; i < c.head_dim; i += 2)
    f.push_back(1.0f / std::pow(c.theta, (float)i / (float)c.head_dim));      // rope.rs:22-25
  if (!c.scaled) return f;                                                      // rope.rs:47
  const float low_wl = c.original_max_positions / c.low_freq_factor;            // rope.rs:30-32
  const float high_wl = c.original_max_positions / c.high_freq_factor;
  for (float& v : f) {                                                          // rope.rs:33-45
    const float wl = 2.0f * 3.14159265358979323846f / v;
    if (wl < high_wl) continue;
    if (wl > low_wl) {
      v = v / c.factor;
    } else {
      const float smooth = (c.original_max_positions / wl - c.low_freq_factor) /
                           (c.high_freq_factor - c.low_freq_factor);
      v = (1.0f - smooth) * v / c.factor + smooth * v;
    }
  }
  return f;
}

// Rotate-half at absolute position p: dim j pairs with j + d/2, angle = float32(p) * f_j in
// float32 (rope.rs:5-8, 61-78, 111-117).
void rotate(float* head, int d, int position, const std::vector<float>& f) {
  const int half = d / 2;
  for (int j = 0; j < half; ++j) {
    const float angle = (float)position * f[j];
    const float c = std::cos(angle), s = std::sin(angle);
    const float a = head[j], b = head[j + half];
    head[j] = a * c - b * s;
    head[j + half] = b * c + a * s;
  }
}

}  // namespace

// Logits (n, vocab) of one whole sequence (crates/model/src/llama.rs:218-273, 306-311).
extern "C" __attribute__((visibility("default"))) int plain_host_forward(
    const PlainConfig* cfg, const float* embed, const PlainLayer* layers, const float* final_norm,
    const float* lm_head, const int* ids, int n, float* logits) {
  const PlainConfig& c = *cfg;
  const int H = c.hidden, nh = c.heads, nkv = c.kv_heads, d = c.head_dim, I = c.intermediate;
  if (n <= 0 || nh % nkv != 0 || d % 2 != 0) return 1;
  const int group = nh / nkv;                       // query head h uses KV head h / group
  const std::vector<float> freqs = inverse_frequencies(c);
  const float scale = 1.0f / std::sqrt((float)d);   // attention.rs:147, 210
  std::vector<float> x((size_t)n * H), h(H), q((size_t)n * nh * d), k((size_t)n * nkv * d),
      v((size_t)n * nkv * d), att((size_t)nh * d), proj(H), gate(I), up(I), score(n);
  for (int t = 0; t < n; ++t) {                     // x[t] = E[ids[t]], no scaling (llama.rs:256-262)
    if (ids[t] < 0 || ids[t] >= c.vocab) return 2;
    for (int i = 0; i < H; ++i) x[(size_t)t * H + i] = embed[(long long)ids[t] * H + i];
  }
  for (int l = 0; l < c.layers; ++l) {
    const PlainLayer& w = layers[l];
    // q, k, v of every position, q and k rotated by the position (attention.rs:73-93)
    for (int t = 0; t < n; ++t) {
      rms_norm(&x[(size_t)t * H], w.input_norm, c.eps, H, h.data());           // llama.rs:265
      linear(h.data(), w.q, H, nh * d, &q[(size_t)t * nh * d]);
      linear(h.data(), w.k, H, nkv * d, &k[(size_t)t * nkv * d]);
      linear(h.data(), w.v, H, nkv * d, &v[(size_t)t * nkv * d]);
      for (int hh = 0; hh < nh; ++hh) rotate(&q[((size_t)t * nh + hh) * d], d, t, freqs);
      for (int hh = 0; hh < nkv; ++hh) rotate(&k[((size_t)t * nkv + hh) * d], d, t, freqs);
    }
    // position t sees positions 0..t (attention.rs:225-233); softmax over them in float32
    // with a float64 denominator (attention.rs:219); heads merged head-major (98-101)
    for (int t = 0; t < n; ++t) {
      for (int hh = 0; hh < nh; ++hh) {
        const float* qv = &q[((size_t)t * nh + hh) * d];
        const int kvh = hh / group;                                              // attention.rs:166-171
        float top = -INFINITY;
        for (int u = 0; u <= t; ++u) {
          const float* kv = &k[((size_t)u * nkv + kvh) * d];
          double s = 0.0;
          for (int j = 0; j < d; ++j) s += (double)qv[j] * kv[j];
          score[u] = (float)s * scale;
          top = std::fmax(top, score[u]);
        }
        double denom = 0.0;
        for (int u = 0; u <= t; ++u) {
          score[u] = std::exp(score[u] - top);
          denom += score[u];
        }
        for (int j = 0; j < d; ++j) {
          double s = 0.0;
          for (int u = 0; u <= t; ++u) s += (double)score[u] * v[((size_t)u * nkv + kvh) * d + j];
          att[(size_t)hh * d + j] = (float)(s / denom);
        }
      }
      linear(att.data(), w.o, nh * d, H, proj.data());                           // attention.rs:102
      for (int i = 0; i < H; ++i) x[(size_t)t * H + i] += proj[i];               // llama.rs:267
    }
    // x += down(silu(gate(y)) * up(y)), silu(z) = z / (1 + e^-z) (layers.rs:179-186)
    for (int t = 0; t < n; ++t) {
      rms_norm(&x[(size_t)t * H], w.post_norm, c.eps, H, h.data());             // llama.rs:268
      linear(h.data(), w.gate, H, I, gate.data());
      linear(h.data(), w.up, H, I, up.data());
      for (int i = 0; i < I; ++i) gate[i] = gate[i] / (1.0f + std::exp(-gate[i])) * up[i];
      linear(gate.data(), w.down, I, H, proj.data());
      for (int i = 0; i < H; ++i) x[(size_t)t * H + i] += proj[i];               // llama.rs:270
    }
  }
  for (int t = 0; t < n; ++t) {                                                 // llama.rs:272-285
    rms_norm(&x[(size_t)t * H], final_norm, c.eps, H, h.data());
    linear(h.data(), c.tied ? embed : lm_head, H, c.vocab, &logits[(size_t)t * c.vocab]);
  }
  return 0;
}
