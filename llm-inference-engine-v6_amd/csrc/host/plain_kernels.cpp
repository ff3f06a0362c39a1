// Plain C++ twins of the device kernels: one serial 32-bit loop nest per operation, in the
// order in which the reference's scalar kernels evaluate them. Nothing on the product path
// calls these; the tests call them through the host library's C interface and hold every
// device kernel, and the tests' own plain Python implementation, against them.
//
// Shapes follow the device kernels: weights are [out, in] row-major and y = x W^T, without
// biases (the reference's src/kernels.hpp:6-7); a head is a contiguous slice of a row.
#include <cmath>
#include <cstdint>
#include <vector>

#include "host_api.h"

extern "C" {

// h = E[token, :], a row copy without scaling (src/kernels.cpp:59-66).
int llme_plain_embed(const float* table, const int32_t* tokens, int T, int V, int H, float* out) {
    if (T < 0 || V <= 0 || H <= 0) return LLME_HOST_BAD_ARGUMENT;
    for (int t = 0; t < T; ++t) {
        if (tokens[t] < 0 || tokens[t] >= V) return LLME_HOST_BAD_ARGUMENT;
        const float* row = table + static_cast<size_t>(tokens[t]) * H;
        for (int i = 0; i < H; ++i) out[static_cast<size_t>(t) * H + i] = row[i];
    }
    return 0;
}

// ss = sum x_i^2 (serial, 32-bit); inv = 1 / sqrt(ss / H + eps); y_i = (w_i * x_i) * inv
// (src/kernels.cpp:18-24).
int llme_plain_rmsnorm(const float* x, const float* w, int T, int H, float eps, float* out) {
    if (T < 0 || H <= 0) return LLME_HOST_BAD_ARGUMENT;
    for (int t = 0; t < T; ++t) {
        const float* row = x + static_cast<size_t>(t) * H;
        float ss = 0.0f;
        for (int i = 0; i < H; ++i) ss += row[i] * row[i];
        const float inv = 1.0f / std::sqrt(ss / static_cast<float>(H) + eps);
        for (int i = 0; i < H; ++i) out[static_cast<size_t>(t) * H + i] = (w[i] * row[i]) * inv;
    }
    return 0;
}

// out[m, n] (+)= sum_k a[m, k] * w[n, k] (src/kernels.cpp:33-57).
int llme_plain_linear(const float* a, const float* w, int M, int N, int K, float* out, int accumulate) {
    if (M < 0 || N <= 0 || K <= 0) return LLME_HOST_BAD_ARGUMENT;
    for (int m = 0; m < M; ++m)
        for (int n = 0; n < N; ++n) {
            const float* ar = a + static_cast<size_t>(m) * K;
            const float* wr = w + static_cast<size_t>(n) * K;
            float acc = 0.0f;
            for (int k = 0; k < K; ++k) acc += ar[k] * wr[k];
            float* o = out + static_cast<size_t>(m) * N + n;
            *o = accumulate ? *o + acc : acc;
        }
    return 0;
}

// silu(g) * u with silu(v) = v / (1 + exp(-v)) (src/kernels.cpp:26-31, src/engine.cpp:213-216).
int llme_plain_swiglu(const float* gate, const float* up, size_t n, float* out) {
    for (size_t i = 0; i < n; ++i) out[i] = gate[i] / (1.0f + std::exp(-gate[i])) * up[i];
    return 0;
}

// Inverse frequencies in 64-bit, stored in 32-bit (src/kernels.cpp:114-160). With scaling:
// wavelengths above orig / low are divided by factor, below orig / high kept, between blended.
int llme_plain_inv_freq(int head_dim, double theta, int has_scaling, double factor, double low, double high,
                        double original, float* out) {
    if (head_dim <= 0 || head_dim % 2 != 0 || theta <= 0.0) return LLME_HOST_BAD_ARGUMENT;
    const int half = head_dim / 2;
    const double pi = 3.14159265358979323846;
    for (int i = 0; i < half; ++i) {
        double fr = 1.0 / std::pow(theta, static_cast<double>(2 * i) / static_cast<double>(head_dim));
        if (has_scaling) {
            const double low_wavelen = original / low, high_wavelen = original / high;
            const double wavelen = 2.0 * pi / fr;
            if (wavelen > low_wavelen) {
                fr = fr / factor;
            } else if (!(wavelen < high_wavelen)) {
                const double smooth = (original / wavelen - low) / (high - low);
                fr = (1.0 - smooth) * fr / factor + smooth * fr;
            }
        }
        out[i] = static_cast<float>(fr);
    }
    return 0;
}

// cos, sin [n, head_dim]: angle = p * inv_freq[i] in 64-bit, both halves of a row equal
// (src/kernels.cpp:162-187).
int llme_plain_rope_tables(const float* inv_freq, const int32_t* positions, int n, int head_dim, float* cos_out,
                           float* sin_out) {
    if (n < 0 || head_dim <= 0 || head_dim % 2 != 0) return LLME_HOST_BAD_ARGUMENT;
    const int half = head_dim / 2;
    for (int r = 0; r < n; ++r)
        for (int i = 0; i < half; ++i) {
            const double angle = static_cast<double>(positions[r]) * static_cast<double>(inv_freq[i]);
            const float c = static_cast<float>(std::cos(angle)), s = static_cast<float>(std::sin(angle));
            cos_out[static_cast<size_t>(r) * head_dim + i] = cos_out[static_cast<size_t>(r) * head_dim + i + half] = c;
            sin_out[static_cast<size_t>(r) * head_dim + i] = sin_out[static_cast<size_t>(r) * head_dim + i + half] = s;
        }
    return 0;
}

// x [T, heads, hd] in place, cos/sin [T, hd]; pairs are (i, i + hd/2):
// x[i] <- a cos[i] - b sin[i]; x[i + hd/2] <- b cos[i + hd/2] + a sin[i + hd/2]
// (src/kernels.cpp:189-203).
int llme_plain_rope_apply(float* x, const float* cos_t, const float* sin_t, int T, int heads, int head_dim) {
    if (T < 0 || heads <= 0 || head_dim <= 0 || head_dim % 2 != 0) return LLME_HOST_BAD_ARGUMENT;
    const int half = head_dim / 2;
    for (int t = 0; t < T; ++t)
        for (int h = 0; h < heads; ++h) {
            float* v = x + (static_cast<size_t>(t) * heads + h) * head_dim;
            const float* c = cos_t + static_cast<size_t>(t) * head_dim;
            const float* s = sin_t + static_cast<size_t>(t) * head_dim;
            for (int i = 0; i < half; ++i) {
                const float a = v[i], b = v[i + half];
                v[i] = a * c[i] - b * s[i];
                v[i + half] = b * c[i + half] + a * s[i + half];
            }
        }
    return 0;
}

// One request: q [T, n_q, hd] are the queries of positions ctx .. ctx + T - 1, k and v
// [ctx + T, n_kv, hd] all keys and values so far. Query head h reads kv head h / (n_q / n_kv);
// s_t = (q . K[t]) * hd^-1/2 for t <= position (and t > position - window if window > 0);
// m = max s; p_t = exp(s_t - m); out = sum_t (p_t / sum p) V[t] (src/kernels.cpp:413-474).
int llme_plain_attention(const float* q, const float* k, const float* v, int T, int ctx, int n_q, int n_kv,
                         int head_dim, int window, float* out) {
    if (T < 0 || ctx < 0 || n_q <= 0 || n_kv <= 0 || n_q % n_kv != 0 || head_dim <= 0 || window < 0)
        return LLME_HOST_BAD_ARGUMENT;
    const int group = n_q / n_kv;
    const float scale = 1.0f / std::sqrt(static_cast<float>(head_dim));
    std::vector<float> scores(static_cast<size_t>(ctx) + T);
    for (int r = 0; r < T; ++r) {
        const int pos = ctx + r;
        const int lo = window > 0 && pos - window + 1 > 0 ? pos - window + 1 : 0;
        for (int h = 0; h < n_q; ++h) {
            const int kv_h = h / group;
            const float* qv = q + (static_cast<size_t>(r) * n_q + h) * head_dim;
            float m = -INFINITY;
            for (int t = lo; t <= pos; ++t) {
                const float* kv = k + (static_cast<size_t>(t) * n_kv + kv_h) * head_dim;
                float dot = 0.0f;
                for (int i = 0; i < head_dim; ++i) dot += qv[i] * kv[i];
                scores[t] = dot * scale;
                if (scores[t] > m) m = scores[t];
            }
            float denom = 0.0f;
            for (int t = lo; t <= pos; ++t) {
                scores[t] = std::exp(scores[t] - m);
                denom += scores[t];
            }
            const float inv = 1.0f / denom;
            float* o = out + (static_cast<size_t>(r) * n_q + h) * head_dim;
            for (int i = 0; i < head_dim; ++i) o[i] = 0.0f;
            for (int t = lo; t <= pos; ++t) {
                const float p = scores[t] * inv;
                const float* vv = v + (static_cast<size_t>(t) * n_kv + kv_h) * head_dim;
                for (int i = 0; i < head_dim; ++i) o[i] += p * vv[i];
            }
        }
    }
    return 0;
}

// First index of the maximum, strict > (src/engine.cpp:52-58).
int llme_plain_argmax(const float* row, int V) {
    if (V <= 0) return LLME_HOST_BAD_ARGUMENT;
    int arg = 0;
    float best = row[0];
    for (int i = 1; i < V; ++i)
        if (row[i] > best) {
            best = row[i];
            arg = i;
        }
    return arg;
}

// Temperature sampling: p = exp((row - max) / T); the token is the first id (ascending) whose
// cumulative sum exceeds u * sum(p); the last id with p > 0 if rounding leaves none. The
// reference has no sampler besides the argmax; this states the device kernel's rule serially,
// with the sums in 64-bit so that the tests can bound the device's 32-bit rounding.
int llme_plain_sample(const float* row, int V, float temperature, float u) {
    if (V <= 0 || !(temperature > 0.0f)) return LLME_HOST_BAD_ARGUMENT;
    float m = row[0];
    for (int i = 1; i < V; ++i)
        if (row[i] > m) m = row[i];
    double total = 0.0;
    for (int i = 0; i < V; ++i) total += std::exp((static_cast<double>(row[i]) - m) / temperature);
    const double target = static_cast<double>(u) * total;
    double cum = 0.0;
    int last = 0;
    for (int i = 0; i < V; ++i) {
        const double p = std::exp((static_cast<double>(row[i]) - m) / temperature);
        if (p > 0.0) last = i;
        cum += p;
        if (cum > target) return i;
    }
    return last;
}

}  // extern "C"
