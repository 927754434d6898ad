// TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's TurboQuant KV-cache codec and of
// attention over quantized K / V rows.  Nothing in the product may include, link or call this.
//
// Follows crates/compute/src/kv_quant.rs (sign vector :54-81, randomized Hadamard transform :90-107,
// Lloyd-Max codebook :115-256, midpoints / index :262-273, LSB-first packing :276-334, row codec
// :340-382), crates/compute/src/wht.rs:5-29 and crates/compute/src/kv_quant_attention.rs:46-136.
//
// Pinned by the reference's own fixture crates/compute/tests/generated/kv_quant_oracle.rs (sign
// vectors, codebooks, input rows, norms and packed words of four (dim, bits) shapes; the checks of
// crates/compute/tests/kv_quant.rs:447-505) and by the laws of that test file (codebook sorted,
// symmetric and bounded; index == nearest centroid; packing round trips and straddles words;
// the inverse rotation undoes the forward one; attention over quantized rows == attention over the
// dequantized rows; sinks enter the denominator only).
#include <algorithm>
#include <cmath>
#include <cstdint>
#include <cstring>
#include <vector>

#include "tsoracle.h"

namespace {

// kv_quant.rs:54-60
uint64_t splitmix64_next(uint64_t& state) {
    state += 0x9E3779B97F4A7C15ull;
    uint64_t z = state;
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    return z ^ (z >> 31);
}

// wht.rs:15-29: the recursion pairs i with i + n/2 after transforming both halves, every stage scaled
// by 1/sqrt(2) -- bottom-up here, the same operations on the same operands
void wht(const float* x, int n, float* y) {
    std::vector<float> a(x, x + n), b((size_t)n);
    const float inv_sqrt2 = 1.0f / std::sqrt(2.0f);
    for (int len = 2; len <= n; len <<= 1) {
        const int half = len / 2;
        for (int blk = 0; blk < n; blk += len)
            for (int i = 0; i < half; i++) {
                const float lo = a[blk + i], hi = a[blk + half + i];
                b[blk + i] = (lo + hi) * inv_sqrt2;
                b[blk + half + i] = (lo - hi) * inv_sqrt2;
            }
        a.swap(b);
    }
    std::memcpy(y, a.data(), (size_t)n * sizeof(float));
}

// kv_quant.rs:115-121
double beta_log_density(double x, int dim) {
    if (dim <= 1) return 0.0;
    const double one_minus_x2 = std::max(1.0 - x * x, 1e-30);
    return (((double)dim - 3.0) / 2.0) * std::log(one_minus_x2);
}

// kv_quant.rs:126-148 (np.interp)
double interp(double q, const std::vector<double>& cdf, const std::vector<double>& grid) {
    if (std::isnan(q)) return NAN;
    if (q <= cdf.front()) return grid.front();
    if (q >= cdf.back()) return grid.back();
    const size_t idx = (size_t)(std::lower_bound(cdf.begin(), cdf.end(), q) - cdf.begin());  // first cdf[idx] >= q
    if (cdf[idx] == q) return grid[idx];
    const double x0 = cdf[idx - 1], x1 = cdf[idx], y0 = grid[idx - 1], y1 = grid[idx];
    if (x1 == x0) return y0;
    return y0 + (y1 - y0) * (q - x0) / (x1 - x0);
}

uint32_t quantize_index(float value, const float* midpoints, int n_mid) {
    uint32_t c = 0;
    for (int i = 0; i < n_mid; i++) c += value > midpoints[i] ? 1u : 0u;
    return c;
}

}  // namespace

extern "C" {

// kv_quant.rs:68-81
void tso_tq_sign_vector(int dim, uint64_t seed, float* out) {
    uint64_t state = seed + (uint64_t)dim * 7919ull;
    for (int i = 0; i < dim; i++) out[i] = (splitmix64_next(state) & 1ull) == 0 ? -1.0f : 1.0f;
}

void tso_tq_wht(const float* x, int n, float* y) { wht(x, n, y); }

// kv_quant.rs:90-107
void tso_tq_rht_forward(const float* x, const float* signs, int n, float* y) {
    std::vector<float> t((size_t)n);
    for (int i = 0; i < n; i++) t[i] = x[i] * signs[i];
    wht(t.data(), n, y);
}
void tso_tq_rht_inverse(const float* x, const float* signs, int n, float* y) {
    wht(x, n, y);
    for (int i = 0; i < n; i++) y[i] = y[i] * signs[i];
}

// kv_quant.rs:166-256; returns the number of levels written
int tso_tq_codebook(int dim, int bits, float* out) {
    if (bits == 0) return 0;
    const int levels = 1 << bits;
    if (dim <= 1) {
        if (levels == 1) {
            out[0] = 0.0f;
            return 1;
        }
        for (int i = 0; i < levels; i++) out[i] = -1.0f + 2.0f * (float)i / ((float)levels - 1.0f);
        return levels;
    }
    const int G = 32768;
    std::vector<double> grid((size_t)G), weights((size_t)G), cdf((size_t)G);
    for (int i = 0; i < G; i++) {
        const double t = (double)i / ((double)G - 1.0);
        grid[i] = (-1.0 + 1e-6) + t * (2.0 - 2e-6);
    }
    double max_log = -INFINITY;
    for (int i = 0; i < G; i++) {
        weights[i] = beta_log_density(grid[i], dim);
        max_log = std::max(max_log, weights[i]);
    }
    double total = 0.0;
    for (int i = 0; i < G; i++) {
        weights[i] = std::exp(weights[i] - max_log);
        total += weights[i];
    }
    if (total > 0.0) {
        for (int i = 0; i < G; i++) weights[i] /= total;
    } else {
        for (int i = 0; i < G; i++) weights[i] = 1.0 / (double)G;
    }
    double running = 0.0;
    for (int i = 0; i < G; i++) {
        running += weights[i];
        cdf[i] = running;
    }
    std::vector<double> centroids((size_t)levels);
    for (int i = 0; i < levels; i++) centroids[i] = interp(((double)i + 0.5) / (double)levels, cdf, grid);
    for (int it = 0; it < 100; it++) {
        std::vector<double> boundaries((size_t)levels + 1, 0.0);
        boundaries[0] = -1.0;
        boundaries[levels] = 1.0;
        for (int i = 1; i < levels; i++) boundaries[i] = 0.5 * (centroids[i - 1] + centroids[i]);
        std::vector<double> next = centroids;
        for (int i = 0; i < levels; i++) {
            const double lo = boundaries[i], hi = boundaries[i + 1];
            const bool last = i == levels - 1;
            double num = 0.0, den = 0.0;
            for (int g = 0; g < G; g++) {
                const double x = grid[g];
                const bool inside = last ? (x >= lo && x <= hi) : (x >= lo && x < hi);
                if (inside) {
                    num += weights[g] * x;
                    den += weights[g];
                }
            }
            if (den > 0.0) next[i] = num / den;
        }
        double max_delta = 0.0;
        for (int i = 0; i < levels; i++) max_delta = std::max(max_delta, std::fabs(centroids[i] - next[i]));
        centroids = next;
        if (max_delta < 1e-6) break;
    }
    for (int i = 0; i < levels; i++) out[i] = (float)centroids[i];
    return levels;
}

// kv_quant.rs:262-264
void tso_tq_midpoints(const float* codebook, int levels, float* out) {
    for (int i = 0; i + 1 < levels; i++) out[i] = 0.5f * (codebook[i] + codebook[i + 1]);
}

int tso_tq_packed_words(int length, int bits) { return length == 0 || bits == 0 ? 0 : (length * bits + 31) / 32; }

// kv_quant.rs:289-312; returns -1 for an index that does not fit or a width outside 1..16
int tso_tq_pack(const uint32_t* indices, int length, int bits, uint32_t* packed) {
    if (bits == 0) return 0;
    if (bits < 1 || bits > 16) return -1;
    const int width = tso_tq_packed_words(length, bits);
    std::memset(packed, 0, (size_t)width * 4);
    for (int i = 0; i < length; i++) {
        const uint32_t value = indices[i];
        if (value >> bits) return -1;
        const uint32_t bit_offset = (uint32_t)i * (uint32_t)bits;
        const uint32_t w = bit_offset / 32, offset = bit_offset % 32;
        packed[w] |= value << offset;
        const int spill = (int)offset + bits - 32;
        if (spill > 0) packed[w + 1] |= value >> (bits - spill);
    }
    return width;
}

// kv_quant.rs:315-334
int tso_tq_unpack(const uint32_t* packed, int bits, int length, uint32_t* indices) {
    if (bits == 0) return 0;
    if (bits < 1 || bits > 16) return -1;
    const uint32_t mask = (1u << bits) - 1u;
    for (int i = 0; i < length; i++) {
        const uint32_t bit_offset = (uint32_t)i * (uint32_t)bits;
        const uint32_t w = bit_offset / 32, offset = bit_offset % 32;
        uint32_t value = packed[w] >> offset;
        const int spill = (int)offset + bits - 32;
        if (spill > 0) value |= packed[w + 1] << (bits - spill);
        indices[i] = value & mask;
    }
    return length;
}

// kv_quant.rs:349-362: norm = ||x|| (f32 sum of squares in index order), unit = x * (1 / max(norm, eps)),
// rotated, one index per coordinate, packed
void tso_tq_quantize_row(const float* x, int dim, const float* signs, const float* midpoints, int bits, float* norm_out,
                         uint32_t* words) {
    float ss = 0.0f;
    for (int i = 0; i < dim; i++) ss += x[i] * x[i];
    const float norm = std::sqrt(ss);
    const float inv = 1.0f / std::max(norm, 1e-6f);
    std::vector<float> unit((size_t)dim), rot((size_t)dim);
    for (int i = 0; i < dim; i++) unit[i] = x[i] * inv;
    tso_tq_rht_forward(unit.data(), signs, dim, rot.data());
    std::vector<uint32_t> idx((size_t)dim);
    const int n_mid = (1 << bits) - 1;
    for (int i = 0; i < dim; i++) idx[i] = quantize_index(rot[i], midpoints, n_mid);
    tso_tq_pack(idx.data(), dim, bits, words);
    *norm_out = norm;
}

// kv_quant.rs:367-379
void tso_tq_dequantize_row(float norm, const uint32_t* words, const float* signs, const float* codebook, int bits, int dim,
                           float* out) {
    std::vector<uint32_t> idx((size_t)dim);
    tso_tq_unpack(words, bits, dim, idx.data());
    std::vector<float> rot((size_t)dim);
    for (int i = 0; i < dim; i++) rot[i] = codebook[idx[i]];
    tso_tq_rht_inverse(rot.data(), signs, dim, out);
    for (int i = 0; i < dim; i++) out[i] = out[i] * norm;
}

// n rows of `dim` values through quantize_row and dequantize_row: what a quantized layer's cache holds of them
void tso_tq_roundtrip_rows(const float* x, int64_t n, int dim, const float* signs, const float* codebook, const float* midpoints,
                           int bits, float* out) {
    std::vector<uint32_t> words((size_t)tso_tq_packed_words(dim, bits) + 1);
    for (int64_t r = 0; r < n; r++) {
        float norm;
        tso_tq_quantize_row(x + r * dim, dim, signs, midpoints, bits, &norm, words.data());
        tso_tq_dequantize_row(norm, words.data(), signs, codebook, bits, dim, out + r * dim);
    }
}

// kv_quant_attention.rs:58-136: one query position over seq_len quantized rows.  q: [nq][hd]; k / v words:
// [seq_len][nkv][words per row], norms [seq_len][nkv]; scale <= 0: 1 / sqrt(hd); sinks nullable [nq].  The two
// sides carry their own tables and widths (kv_quant_attention.rs:24-44).
void tso_tq_attention(const float* q, const uint32_t* k_words, const float* k_norms, const uint32_t* v_words,
                      const float* v_norms, int hd, int nq, int nkv, int seq_len, float scale, const float* sinks,
                      const float* k_signs, const float* k_codebook, const float* v_signs, const float* v_codebook, int k_bits,
                      int v_bits, float* out) {
    const int group = nq / nkv, k_wpr = tso_tq_packed_words(hd, k_bits), v_wpr = tso_tq_packed_words(hd, v_bits);
    if (!(scale > 0.0f)) scale = 1.0f / std::sqrt((float)hd);
    std::vector<float> q_rot((size_t)hd), scores((size_t)seq_len), acc_rot((size_t)hd), acc((size_t)hd);
    std::vector<uint32_t> idx((size_t)hd);
    for (int qh = 0; qh < nq; qh++) {
        const int kvh = qh / group;
        tso_tq_rht_forward(q + (size_t)qh * hd, k_signs, hd, q_rot.data());
        for (int p = 0; p < seq_len; p++) {
            const size_t row = (size_t)p * nkv + kvh;
            tso_tq_unpack(k_words + row * k_wpr, k_bits, hd, idx.data());
            float dot = 0.0f;
            for (int d = 0; d < hd; d++) dot += q_rot[d] * k_codebook[idx[d]];
            scores[p] = dot * k_norms[row] * scale;
        }
        float mx = -INFINITY;
        for (int p = 0; p < seq_len; p++) mx = std::max(mx, scores[p]);
        if (sinks) mx = std::max(mx, sinks[qh]);
        for (int p = 0; p < seq_len; p++) scores[p] = std::exp(scores[p] - mx);
        float sum = 0.0f;
        for (int p = 0; p < seq_len; p++) sum += scores[p];
        if (sinks) sum += std::exp(sinks[qh] - mx);
        const float inv_sum = 1.0f / sum;
        for (int p = 0; p < seq_len; p++) scores[p] *= inv_sum;
        std::fill(acc_rot.begin(), acc_rot.end(), 0.0f);
        for (int p = 0; p < seq_len; p++) {
            const size_t row = (size_t)p * nkv + kvh;
            tso_tq_unpack(v_words + row * v_wpr, v_bits, hd, idx.data());
            const float coeff = scores[p] * v_norms[row];
            for (int d = 0; d < hd; d++) acc_rot[d] += coeff * v_codebook[idx[d]];
        }
        tso_tq_rht_inverse(acc_rot.data(), v_signs, hd, acc.data());
        std::memcpy(out + (size_t)qh * hd, acc.data(), (size_t)hd * sizeof(float));
    }
}

}  // extern "C"
