// The plain backend of the whole model: a Llama decoder over one whole sequence, in serial 32-bit
// loops, put together from the plain kernels of plain_kernels.cpp in the order of the reference's
// forward pass (src/engine.cpp:105-261, there one token at a time against a cache; here all T
// tokens of the sequence at once, which read their own keys and values, so there is no cache to
// get wrong). Nothing on the product path calls it: it is what the device's 32-bit path, and the
// tests' plain Python implementation, are held against as a whole.
#include <cstdint>
#include <cstddef>
#include <vector>

#include "host_api.h"

extern "C" {

int llme_plain_embed(const float* table, const int32_t* tokens, int T, int V, int H, float* out);
int llme_plain_rmsnorm(const float* x, const float* w, int T, int H, float eps, float* out);
int llme_plain_linear(const float* a, const float* w, int M, int N, int K, float* out, int accumulate);
int llme_plain_swiglu(const float* gate, const float* up, size_t n, float* out);
int llme_plain_inv_freq(int head_dim, double theta, int has_scaling, double factor, double low, double high,
                        double original_max, float* out);
int llme_plain_rope_tables(const float* inv_freq, const int32_t* positions, int n, int head_dim, float* cos_out,
                           float* sin_out);
int llme_plain_rope_apply(float* x, const float* cos_t, const float* sin_t, int T, int heads, int head_dim);
int llme_plain_attention(const float* q, const float* k, const float* v, int T, int ctx, int n_q, int n_kv,
                         int head_dim, int window, float* out);

// sizes: {layers, hidden, intermediate, query heads, kv heads, head size, vocabulary, window}
// rope: {theta, has_scaling, factor, low_freq_factor, high_freq_factor, original_max_position}
// layer_weights: 9 pointers a layer, in the order input norm [H], q [n_q hd, H], k [n_kv hd, H],
// v [n_kv hd, H], o [H, n_q hd], post-attention norm [H], gate [F, H], up [F, H], down [H, F];
// embed [V, H]; final_norm [H]; head [V, H] (the embedding again where the head is tied,
// src/model.cpp:185-195). tokens, positions [T]; logits [T, V].
int llme_plain_llama_forward(const int32_t* sizes, const double* rope, float eps, const float* embed,
                             const float* final_norm, const float* head, const float* const* layer_weights,
                             const int32_t* tokens, const int32_t* positions, int T, float* logits) {
    if (!sizes || !rope || !embed || !final_norm || !head || !layer_weights || !tokens || !positions || !logits)
        return LLME_HOST_BAD_ARGUMENT;
    const int L = sizes[0], H = sizes[1], F = sizes[2], n_q = sizes[3], n_kv = sizes[4], hd = sizes[5], V = sizes[6];
    const int window = sizes[7];
    if (T <= 0 || L < 0 || H <= 0 || F <= 0 || n_q <= 0 || n_kv <= 0 || hd <= 0 || hd % 2 != 0 || V <= 0)
        return LLME_HOST_BAD_ARGUMENT;
    const size_t t = static_cast<size_t>(T);
    const int QD = n_q * hd, KD = n_kv * hd;
    std::vector<float> inv(hd / 2), cos_t(t * hd), sin_t(t * hd);
    int rc = llme_plain_inv_freq(hd, rope[0], rope[1] != 0.0 ? 1 : 0, rope[2], rope[3], rope[4], rope[5], inv.data());
    if (rc < 0) return rc;
    rc = llme_plain_rope_tables(inv.data(), positions, T, hd, cos_t.data(), sin_t.data());
    if (rc < 0) return rc;

    std::vector<float> h(t * H), x(t * H), q(t * QD), k(t * KD), v(t * KD), attn(t * QD), gate(t * F), up(t * F),
        act(t * F);
    rc = llme_plain_embed(embed, tokens, T, V, H, h.data());                                   // engine.cpp:118
    if (rc < 0) return rc;
    for (int l = 0; l < L; ++l) {
        const float* const* w = layer_weights + static_cast<size_t>(l) * 9;
        for (int i = 0; i < 9; ++i)
            if (!w[i]) return LLME_HOST_BAD_ARGUMENT;
        llme_plain_rmsnorm(h.data(), w[0], T, H, eps, x.data());                               // engine.cpp:137
        llme_plain_linear(x.data(), w[1], T, QD, H, q.data(), 0);                              // engine.cpp:142-144
        llme_plain_linear(x.data(), w[2], T, KD, H, k.data(), 0);
        llme_plain_linear(x.data(), w[3], T, KD, H, v.data(), 0);
        llme_plain_rope_apply(q.data(), cos_t.data(), sin_t.data(), T, n_q, hd);               // engine.cpp:163-170
        llme_plain_rope_apply(k.data(), cos_t.data(), sin_t.data(), T, n_kv, hd);
        rc = llme_plain_attention(q.data(), k.data(), v.data(), T, 0, n_q, n_kv, hd, window, attn.data());   // 186-189
        if (rc < 0) return rc;
        llme_plain_linear(attn.data(), w[4], T, H, QD, h.data(), 1);                           // engine.cpp:193,206
        llme_plain_rmsnorm(h.data(), w[5], T, H, eps, x.data());                               // engine.cpp:208
        llme_plain_linear(x.data(), w[6], T, F, H, gate.data(), 0);                            // engine.cpp:213-216
        llme_plain_linear(x.data(), w[7], T, F, H, up.data(), 0);
        llme_plain_swiglu(gate.data(), up.data(), t * F, act.data());
        llme_plain_linear(act.data(), w[8], T, H, F, h.data(), 1);                             // engine.cpp:230-239
    }
    llme_plain_rmsnorm(h.data(), final_norm, T, H, eps, x.data());                             // engine.cpp:243
    return llme_plain_linear(x.data(), head, T, V, H, logits, 0);                              // engine.cpp:247
}

}  // extern "C"
