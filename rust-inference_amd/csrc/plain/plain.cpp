// Plain C++ twins of the kernel families (see plain.h).  Scalar loops in float32, the reference's order.
#include "plain.h"

#include <math.h>
#include <string.h>

#include <algorithm>
#include <vector>

extern "C" uint16_t ri_plain_f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x0040u);      // NaN stays a quiet NaN
    const uint32_t bias = 0x7FFFu + ((u >> 16) & 1u);                                    // ties to even
    return (uint16_t)((u + bias) >> 16);
}

extern "C" float ri_plain_bf16_to_f32(uint16_t b) {
    const uint32_t u = (uint32_t)b << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}

extern "C" int ri_plain_embedding(float* out, const float* table, const int32_t* ids, int tokens, int vocab, int dim) {
    for (int t = 0; t < tokens; ++t) {
        if (ids[t] < 0 || ids[t] >= vocab) return 1;
        memcpy(out + (size_t)t * dim, table + (size_t)ids[t] * dim, sizeof(float) * (size_t)dim);
    }
    return 0;
}

extern "C" void ri_plain_rms_norm(float* out, const float* x, const float* gain, int rows, int dim, float eps) {
    for (int r = 0; r < rows; ++r) {
        const float* xr = x + (size_t)r * dim;
        float ss = 0.f;
        for (int d = 0; d < dim; ++d) ss += xr[d] * xr[d];
        const float inv = 1.0f / sqrtf(ss / (float)dim + eps);
        for (int d = 0; d < dim; ++d) out[(size_t)r * dim + d] = xr[d] * inv * gain[d];
    }
}

extern "C" void ri_plain_add_rms_norm(float* out, float* residual, const float* pending, const float* gain, int rows,
                                      int dim, float eps) {
    for (size_t i = 0; i < (size_t)rows * dim; ++i) residual[i] += pending[i];
    ri_plain_rms_norm(out, residual, gain, rows, dim, eps);
}

extern "C" void ri_plain_rope_inv_freq(float* inv_freq, int rot_dim, float theta) {
    for (int i = 0; i < rot_dim / 2; ++i) inv_freq[i] = 1.0f / powf(theta, (2.0f * (float)i) / (float)rot_dim);
}

extern "C" void ri_plain_rope(float* x, const int32_t* positions, const float* inv_freq, int tokens, int heads,
                              int head_dim, int rot_dim) {
    const int half = rot_dim / 2;
    for (int t = 0; t < tokens; ++t)
        for (int h = 0; h < heads; ++h) {
            float* v = x + ((size_t)t * heads + h) * head_dim;
            for (int i = 0; i < half; ++i) {
                const float angle = (float)positions[t] * inv_freq[i];
                const float c = cosf(angle), s = sinf(angle);
                const float a = v[i], b = v[i + half];
                v[i] = a * c - b * s;
                v[i + half] = b * c + a * s;
            }
        }
}

extern "C" void ri_plain_linear(float* out, const float* x, const float* w, int m, int n, int k) {
    for (int i = 0; i < m; ++i)
        for (int j = 0; j < n; ++j) {
            float acc = 0.f;
            for (int p = 0; p < k; ++p) acc += x[(size_t)i * k + p] * w[(size_t)j * k + p];
            out[(size_t)i * n + j] = acc;
        }
}

extern "C" void ri_plain_swiglu(float* out, const float* y, int tokens, int inter) {
    for (int t = 0; t < tokens; ++t)
        for (int i = 0; i < inter; ++i) {
            const float g = y[(size_t)t * 2 * inter + i], u = y[(size_t)t * 2 * inter + inter + i];
            out[(size_t)t * inter + i] = g / (1.0f + expf(-g)) * u;
        }
}

extern "C" void ri_plain_attention(float* out, const float* q, const float* k_pages, const float* v_pages,
                                   const int32_t* tok_pos, const int32_t* tok_seq, const int32_t* page_table,
                                   int table_width, int tokens, int heads, int kv_heads, int head_dim, int page_size,
                                   int window, float scale) {
    const int group = heads / kv_heads;
    std::vector<float> acc((size_t)head_dim);
    for (int t = 0; t < tokens; ++t) {
        const int pos = tok_pos[t];
        const int lo = window > 0 ? std::max(0, pos - window + 1) : 0;
        const int32_t* table = page_table + (size_t)tok_seq[t] * table_width;
        for (int h = 0; h < heads; ++h) {
            const int kvh = h / group;                                   // consecutive query heads share a kv head
            const float* qv = q + ((size_t)t * heads + h) * head_dim;
            float m = -INFINITY, l = 0.f;
            std::fill(acc.begin(), acc.end(), 0.f);
            for (int j = lo; j <= pos; ++j) {                            // the mask is the loop's bounds
                const size_t base = ((size_t)table[j / page_size] * kv_heads + kvh) * (size_t)page_size * head_dim;
                const float* kv = k_pages + base + (size_t)(j % page_size) * head_dim;
                float dot = 0.f;
                for (int d = 0; d < head_dim; ++d) dot += qv[d] * kv[d];
                const float s = dot * scale;
                const float m_new = std::max(m, s);
                const float corr = expf(m - m_new), p = expf(s - m_new);  // corr is 0 on the first key
                l = l * corr + p;
                for (int d = 0; d < head_dim; ++d)
                    acc[d] = acc[d] * corr + p * v_pages[base + (size_t)d * page_size + j % page_size];
                m = m_new;
            }
            for (int d = 0; d < head_dim; ++d) out[((size_t)t * heads + h) * head_dim + d] = acc[d] / l;
        }
    }
}

extern "C" int ri_plain_argmax(const float* row, int n) {
    int best = 0;
    for (int i = 1; i < n; ++i)
        if (row[i] > row[best]) best = i;
    return best;
}

extern "C" uint64_t ri_plain_rng_seed(uint64_t seed) {
    uint64_t z = seed + 0x9E3779B97F4A7C15ull;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return (z ^ (z >> 31)) | 1ull;                                       // never zero
}

extern "C" uint64_t ri_plain_rng_next(uint64_t* state) {
    uint64_t x = *state;
    x ^= x >> 12;
    x ^= x << 25;
    x ^= x >> 27;
    *state = x;
    return x * 0x2545F4914F6CDD1Dull;
}

extern "C" float ri_plain_rng_next_f32(uint64_t* state) {
    return (float)(ri_plain_rng_next(state) >> 40) / (float)(1 << 24);  // 24 bits: exact in float32, in [0, 1)
}

extern "C" int ri_plain_sample(const float* logits, int vocab, const int32_t* history, int n_history, float temperature,
                               int top_k, float top_p, float penalty, uint64_t* rng) {
    if (vocab < 1) return -1;
    std::vector<float> row(logits, logits + vocab);
    if (penalty != 1.0f) {
        std::vector<char> seen((size_t)vocab, 0);
        for (int i = 0; i < n_history; ++i)
            if (history[i] >= 0 && history[i] < vocab) seen[history[i]] = 1;
        for (int i = 0; i < vocab; ++i)
            if (seen[i]) row[i] = row[i] > 0.f ? row[i] / penalty : row[i] * penalty;
    }
    if (!(temperature > 0.f)) return ri_plain_argmax(row.data(), vocab);
    struct Cand { int id; float v; };
    std::vector<Cand> cand((size_t)vocab);
    for (int i = 0; i < vocab; ++i) cand[i] = {i, row[i] / temperature};
    // falling value, rising id among equals; the k largest by that order are the first k of the sorted list.
    // Values are compared as the reference compares them (f32::total_cmp, src/sampling.rs:96-101): by a key that
    // orders every bit pattern, NaNs included (a positive NaN above +inf, a negative one below -inf, -0 below +0),
    // so that the comparison is a strict weak ordering whatever the logits hold.
    auto key = [](float v) {
        int32_t b;
        memcpy(&b, &v, sizeof b);
        return b ^ (int32_t)((uint32_t)(b >> 31) >> 1);
    };
    std::sort(cand.begin(), cand.end(), [&key](const Cand& a, const Cand& b) {
        const int32_t ka = key(a.v), kb = key(b.v);
        return ka > kb || (ka == kb && a.id < b.id);
    });
    if (top_k > 0 && top_k < vocab) cand.resize((size_t)top_k);
    std::vector<float> probs(cand.size());
    float total = 0.f;
    for (size_t i = 0; i < cand.size(); ++i) {
        probs[i] = expf(cand[i].v - cand[0].v);
        total += probs[i];
    }
    for (float& p : probs) p /= total;
    if (top_p < 1.0f) {
        float acc = 0.f;
        size_t keep = probs.size();
        for (size_t i = 0; i < probs.size(); ++i) {
            acc += probs[i];
            if (acc >= top_p) { keep = i + 1; break; }
        }
        probs.resize(keep);
        total = 0.f;
        for (float p : probs) total += p;
        for (float& p : probs) p /= total;
    }
    const float r = ri_plain_rng_next_f32(rng);
    float acc = 0.f;
    for (size_t i = 0; i < probs.size(); ++i) {
        acc += probs[i];
        if (r < acc) return cand[i].id;
    }
    return cand[probs.size() - 1].id;
}
