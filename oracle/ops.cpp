// Elementwise / attention / rope operators of the CPU oracle (test infrastructure only).
// Follows crates/compute/src/{rms_norm,rope,attention,gdn}.rs.
#include "tsoracle.h"

#include <cmath>
#include <vector>

// crates/compute/src/rms_norm.rs:5-14
extern "C" void tso_rms_norm(const float* x, const float* w, int64_t n, float eps, float* y) {
    float sum_sq = 0.0f;
    for (int64_t i = 0; i < n; i++) sum_sq += x[i] * x[i];
    float inv_rms = 1.0f / std::sqrt(sum_sq / (float)n + eps);
    for (int64_t i = 0; i < n; i++) y[i] = x[i] * w[i] * inv_rms;
}

static void rotate_pairs(float* x, int num_tokens, int num_heads, int head_dim, int rotated_pairs,
                         const float* cos_t, const float* sin_t) {
    int half = head_dim / 2;
    for (int t = 0; t < num_tokens; t++)
        for (int h = 0; h < num_heads; h++) {
            float* base = x + ((int64_t)t * num_heads + h) * head_dim;
            for (int i = 0; i < rotated_pairs; i++) {
                float x0 = base[i], x1 = base[half + i];
                float c = cos_t[i], s = sin_t[i];
                base[i] = x0 * c - x1 * s;
                base[half + i] = x0 * s + x1 * c;
            }
        }
}

// crates/compute/src/rope.rs:208-256 (NeoX pairs (i, i + head_dim/2); in place here)
extern "C" void tso_rope_neox(float* x, int num_tokens, int num_heads, int head_dim,
                              int rotated_pairs, int64_t position, float theta) {
    float log_theta = std::log(theta);
    float position_f = (float)position;
    std::vector<float> c(rotated_pairs), s(rotated_pairs);
    for (int i = 0; i < rotated_pairs; i++) {
        float exponent = -((float)(2 * i)) / (float)head_dim;
        float angle = position_f * std::exp(exponent * log_theta);
        c[i] = std::cos(angle);
        s[i] = std::sin(angle);
    }
    rotate_pairs(x, num_tokens, num_heads, head_dim, rotated_pairs, c.data(), s.data());
}

// The per-pair angle table variant the Llama-3 flow binds
// (crates/runtime/src/families/llama/attn.rs:325-340, table from rope.rs:447-460):
// angle_i = position * freqs[i], magnitude scale 1.
extern "C" void tso_rope_neox_freqs(float* x, int num_tokens, int num_heads, int head_dim,
                                    int rotated_pairs, int64_t position, const float* freqs) {
    float position_f = (float)position;
    std::vector<float> c(rotated_pairs), s(rotated_pairs);
    for (int i = 0; i < rotated_pairs; i++) {
        float angle = position_f * freqs[i];
        c[i] = std::cos(angle);
        s[i] = std::sin(angle);
    }
    rotate_pairs(x, num_tokens, num_heads, head_dim, rotated_pairs, c.data(), s.data());
}

extern "C" void tso_rope_neox_freqs_scaled(float* x, int num_tokens, int num_heads, int head_dim,
                                           int rotated_pairs, int64_t position, const float* freqs,
                                           float mscale) {
    float position_f = (float)position;
    std::vector<float> c(rotated_pairs), s(rotated_pairs);
    for (int i = 0; i < rotated_pairs; i++) {
        float angle = position_f * freqs[i];
        c[i] = std::cos(angle) * mscale;
        s[i] = std::sin(angle) * mscale;
    }
    rotate_pairs(x, num_tokens, num_heads, head_dim, rotated_pairs, c.data(), s.data());
}

// crates/compute/src/rope.rs:296-372
static float yarn_corr_dim(int n_dims, int64_t n_ctx_orig, float n_rot, float base) {
    return (float)n_dims * std::log((float)n_ctx_orig / (n_rot * 2.0f * 3.14159265358979323846f)) /
           (2.0f * std::log(base));
}
extern "C" void tso_yarn_frequencies(int rotary_dim, float base, float factor, int64_t original_context,
                                     float beta_fast, float beta_slow, float* freqs, float* mscale) {
    const int pairs = rotary_dim / 2;
    const bool active = factor > 0.0f;
    const float freq_scale = active ? 1.0f / factor : 1.0f;
    float low = 0.0f, high = 0.0f;
    if (active) {
        float start = std::floor(yarn_corr_dim(rotary_dim, original_context, beta_fast, base));
        float end = std::ceil(yarn_corr_dim(rotary_dim, original_context, beta_slow, base));
        low = std::fmax(start, 0.0f);
        high = std::fmin(end, (float)rotary_dim - 1.0f);
    }
    for (int p = 0; p < pairs; p++) {
        int i0 = 2 * p;
        float extrap = std::pow(base, -((float)i0) / (float)rotary_dim);
        if (!active) {
            freqs[p] = extrap;
            continue;
        }
        float y = ((float)i0 / 2.0f - low) / std::fmax(high - low, 0.001f);
        float mix = 1.0f - std::fmin(std::fmax(y, 0.0f), 1.0f);
        freqs[p] = extrap * (freq_scale * (1.0f - mix) + mix);
    }
    *mscale = active ? 1.0f + 0.1f * std::log(factor) : 1.0f;
}

// crates/gpu/src/shaders/moe_gguf.metal:528-556
extern "C" float tso_swiglu_oai(float gate, float up, float alpha, float limit) {
    float x = std::fmin(gate, limit);
    float y = std::fmin(std::fmax(up, -limit), limit);
    return (x / (1.0f + std::exp(-alpha * x))) * (y + 1.0f);
}

// crates/compute/src/rope.rs:390-439
extern "C" int tso_llama3_rope_factors(int rotary_dim, double base, double factor,
                                       double low_freq_factor, double high_freq_factor,
                                       double original_context, float* out) {
    bool valid = rotary_dim > 0 && rotary_dim % 2 == 0 && base > 1.0 && factor > 0.0 &&
                 low_freq_factor > 0.0 && high_freq_factor > low_freq_factor &&
                 original_context > 0.0 && std::isfinite(base) && std::isfinite(factor) &&
                 std::isfinite(low_freq_factor) && std::isfinite(high_freq_factor) &&
                 std::isfinite(original_context);
    if (!valid) return -1;
    double low_freq_wavelen = original_context / low_freq_factor;
    double high_freq_wavelen = original_context / high_freq_factor;
    for (int p = 0; p < rotary_dim / 2; p++) {
        double freq = std::pow(base, -((double)(2 * p)) / (double)rotary_dim);
        double wavelen = 2.0 * M_PI / freq;
        double divisor;
        if (wavelen < high_freq_wavelen)
            divisor = 1.0;
        else if (wavelen > low_freq_wavelen)
            divisor = factor;
        else {
            double smooth =
                (original_context / wavelen - low_freq_factor) / (high_freq_factor - low_freq_factor);
            divisor = 1.0 / ((1.0 - smooth) / factor + smooth);
        }
        out[p] = (float)divisor;
    }
    return 0;
}

// crates/compute/src/rope.rs:447-460
extern "C" void tso_rope_frequencies_with_factors(int rotary_dim, float base, const float* factors,
                                                  float* out) {
    for (int p = 0; p < rotary_dim / 2; p++)
        out[p] = std::pow(base, -((float)(2 * p)) / (float)rotary_dim) / factors[p];
}

// crates/compute/src/attention.rs:53-137, with the visited key set generalised from the
// contiguous range [kv_start, seq_len) to "[kv_start, prefix_end) then extra[0..n_extra)":
// the tree-verify attention of crates/gpu/src/attention_decode.rs:1153-1230 (a row sees the
// committed prefix plus the cache slots on its root path).  Same operations in the same
// order; with n_extra == 0 it is the reference function verbatim.
extern "C" void tso_attention_core(const float* q, const float* k, const float* v, int head_dim,
                                   int nq, int nkv, int64_t kv_start, int64_t prefix_end,
                                   const int64_t* extra, int n_extra, float scale,
                                   const float* sinks, float* out) {
    int group = nq / nkv;
    if (!(scale > 0.0f)) scale = 1.0f / std::sqrt((float)head_dim);
    int64_t stride = (int64_t)nkv * head_dim;
    int64_t n_prefix = prefix_end > kv_start ? prefix_end - kv_start : 0;
    std::vector<int64_t> pos((size_t)(n_prefix + n_extra));
    for (int64_t i = 0; i < n_prefix; i++) pos[i] = kv_start + i;
    for (int i = 0; i < n_extra; i++) pos[n_prefix + i] = extra[i];
    std::vector<float> scores(pos.size());
    for (int qh = 0; qh < nq; qh++) {
        int kvh = qh / group;
        const float* qv = q + (int64_t)qh * head_dim;
        for (size_t i = 0; i < pos.size(); i++) {
            const float* kr = k + pos[i] * stride + (int64_t)kvh * head_dim;
            float dot = 0.0f;
            for (int d = 0; d < head_dim; d++) dot += qv[d] * kr[d];
            scores[i] = dot * scale;
        }
        float mx = -INFINITY;
        for (float s : scores) mx = std::fmax(mx, s);
        if (sinks) mx = std::fmax(mx, sinks[qh]);
        for (float& s : scores) s = std::exp(s - mx);
        float sum = 0.0f;
        for (float s : scores) sum += s;
        if (sinks) sum += std::exp(sinks[qh] - mx);
        float inv_sum = 1.0f / sum;
        for (float& s : scores) s *= inv_sum;
        for (int d = 0; d < head_dim; d++) {
            const float* vc = v + (int64_t)kvh * head_dim + d;
            float acc = 0.0f;
            for (size_t i = 0; i < scores.size(); i++) acc += scores[i] * vc[pos[i] * stride];
            out[(int64_t)qh * head_dim + d] = acc;
        }
    }
}

extern "C" void tso_causal_attention(const float* q, const float* k, const float* v, int head_dim,
                                     int nq, int nkv, int64_t seq_len, int64_t window, float scale,
                                     const float* sinks, float* out) {
    int64_t kv_start = 0;
    if (window > 0) kv_start = seq_len > window ? seq_len - window : 0;
    tso_attention_core(q, k, v, head_dim, nq, nkv, kv_start, seq_len, nullptr, 0, scale, sinks, out);
}

// crates/compute/src/gdn.rs:42-44
extern "C" float tso_silu(float x) { return x / (1.0f + std::exp(-x)); }
