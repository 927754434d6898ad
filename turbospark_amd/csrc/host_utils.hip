// Host-side install helpers: GGUF block encoders and the seeded synthetic-weight generator.
//
// The encoders restate the reference's quantize-on-install routines
// (crates/compute/src/quant_gguf/q8_0.rs:56-77, q4_k.rs:126-204); the generator plays the role
// of the reference's random-weight synthetic installs (crates/repack/src/synthetic_*.rs).
#include <algorithm>
#include <cmath>
#include <cstring>
#include <thread>
#include <vector>

#include "tsv_internal.h"

namespace tsv {

static thread_local std::string g_error;
void set_error(const std::string& s) { g_error = s; }
bool error_is_empty() { return g_error.empty(); }
const std::string& get_error() { return g_error; }

int64_t row_bytes(int dtype, int64_t cols) {
    switch (dtype) {
        case TSV_F32: return cols * 4;
        case TSV_F16:
        case TSV_BF16: return cols * 2;
        case TSV_Q8_0: return cols % 32 ? -1 : cols / 32 * 34;
        case TSV_Q4_K: return cols % 256 ? -1 : cols / 256 * 144;
        case TSV_Q5_K: return cols % 256 ? -1 : cols / 256 * 176;
        case TSV_Q6_K: return cols % 256 ? -1 : cols / 256 * 210;
        case TSV_MXFP4: return cols % 32 ? -1 : cols / 32 * 17;
    }
    return -1;
}

namespace {

inline uint16_t f16_bits(float x) {
    _Float16 h = (_Float16)x;  // IEEE round-to-nearest-even
    uint16_t b;
    std::memcpy(&b, &h, 2);
    return b;
}
inline float f16_value(uint16_t b) {
    _Float16 h;
    std::memcpy(&h, &b, 2);
    return (float)h;
}
inline uint16_t bf16_bits(float x) {  // crates/compute/src/quant.rs:28-39
    uint32_t u;
    std::memcpy(&u, &x, 4);
    if (x != x) return (uint16_t)((u >> 16) | 0x40u);
    return (uint16_t)((u + 0x7FFFu + ((u >> 16) & 1u)) >> 16);
}

// Keeps the accumulator on a tie, so +-0 folds to the accumulator's sign.
inline float keep_max(float acc, float v) { return v > acc ? v : acc; }
inline float keep_min(float acc, float v) { return v < acc ? v : acc; }
inline uint8_t round_clamp_u8(float v, float hi) {
    float r = roundf(v);  // half away from zero, as Rust's f32::round
    if (!(r > 0.0f)) return 0;
    return (uint8_t)(r > hi ? hi : r);
}

void encode_q8_0(const float* row, int64_t n, uint8_t* out) {
    for (int64_t b = 0; b < n / 32; b++, row += 32, out += 34) {
        float amax = 0.0f;
        for (int i = 0; i < 32; i++) amax = keep_max(amax, fabsf(row[i]));
        const uint16_t db = f16_bits(amax / 127.0f);
        const float d = f16_value(db);
        const float inv = d == 0.0f ? 0.0f : 1.0f / d;
        std::memcpy(out, &db, 2);
        for (int i = 0; i < 32; i++) {
            int q = (int)roundf(row[i] * inv);
            q = q < -127 ? -127 : q > 127 ? 127 : q;
            out[2 + i] = (uint8_t)(int8_t)q;
        }
    }
}

inline void unpack_scale_min(const uint8_t* p, int j, int& sc, int& mn) {  // q4_k.rs:43-54
    if (j < 4) {
        sc = p[j] & 63;
        mn = p[j + 4] & 63;
    } else {
        sc = (p[j + 4] & 0xF) | ((p[j - 4] >> 6) << 4);
        mn = (p[j + 4] >> 4) | ((p[j] >> 6) << 4);
    }
}

void encode_q4_k(const float* row, int64_t n, uint8_t* out) {
    for (int64_t b = 0; b < n / 256; b++, row += 256, out += 144) {
        float scale[8], mn[8], smax = 0.0f, mmax = 0.0f;
        for (int j = 0; j < 8; j++) {
            const float* s = row + 32 * j;
            float lo = 0.0f;
            for (int i = 0; i < 32; i++) lo = keep_min(lo, s[i]);
            float hi = lo;
            for (int i = 0; i < 32; i++) hi = keep_max(hi, s[i]);
            scale[j] = (hi - lo) / 15.0f;
            mn[j] = -lo;
            smax = keep_max(smax, scale[j]);
            mmax = keep_max(mmax, mn[j]);
        }
        const float is = smax > 0.0f ? 63.0f / smax : 0.0f;
        const float im = mmax > 0.0f ? 63.0f / mmax : 0.0f;
        uint8_t* packed = out + 4;
        std::memset(packed, 0, 12);
        for (int j = 0; j < 8; j++) {
            const uint8_t ls = round_clamp_u8(scale[j] * is, 63.0f), lm = round_clamp_u8(mn[j] * im, 63.0f);
            if (j < 4) {
                packed[j] |= ls;
                packed[j + 4] |= lm;
            } else {
                packed[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                packed[j - 4] |= (uint8_t)((ls >> 4) << 6);
                packed[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        const uint16_t db = f16_bits(smax / 63.0f), mb = f16_bits(mmax / 63.0f);
        std::memcpy(out, &db, 2);
        std::memcpy(out + 2, &mb, 2);
        const float d = f16_value(db), dmin = f16_value(mb);
        uint8_t q[256];
        std::memset(q, 0, sizeof q);
        for (int j = 0; j < 8; j++) {  // quants from the scales as a decoder will read them back
            int sc, m;
            unpack_scale_min(packed, j, sc, m);
            const float step = d * (float)sc;
            if (step == 0.0f) continue;
            const float bias = dmin * (float)m;
            for (int i = 0; i < 32; i++) q[32 * j + i] = round_clamp_u8((row[32 * j + i] + bias) / step, 15.0f);
        }
        for (int g = 0; g < 4; g++)
            for (int l = 0; l < 32; l++) out[16 + 32 * g + l] = (uint8_t)(q[64 * g + l] | (q[64 * g + 32 + l] << 4));
    }
}

// Q5_K: the reference only decodes it (crates/compute/src/quant_gguf/q5_k.rs:47-96); this encoder is
// Q4_K's fitter with 31 levels per sub-block, for synthetic weights in that format.
void encode_q5_k(const float* row, int64_t n, uint8_t* out) {
    for (int64_t b = 0; b < n / 256; b++, row += 256, out += 176) {
        float scale[8], mn[8], smax = 0.0f, mmax = 0.0f;
        for (int j = 0; j < 8; j++) {
            const float* s = row + 32 * j;
            float lo = 0.0f;
            for (int i = 0; i < 32; i++) lo = keep_min(lo, s[i]);
            float hi = lo;
            for (int i = 0; i < 32; i++) hi = keep_max(hi, s[i]);
            scale[j] = (hi - lo) / 31.0f;
            mn[j] = -lo;
            smax = keep_max(smax, scale[j]);
            mmax = keep_max(mmax, mn[j]);
        }
        const float is = smax > 0.0f ? 63.0f / smax : 0.0f;
        const float im = mmax > 0.0f ? 63.0f / mmax : 0.0f;
        uint8_t* packed = out + 4;
        std::memset(packed, 0, 12);
        for (int j = 0; j < 8; j++) {
            const uint8_t ls = round_clamp_u8(scale[j] * is, 63.0f), lm = round_clamp_u8(mn[j] * im, 63.0f);
            if (j < 4) {
                packed[j] |= ls;
                packed[j + 4] |= lm;
            } else {
                packed[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                packed[j - 4] |= (uint8_t)((ls >> 4) << 6);
                packed[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        const uint16_t db = f16_bits(smax / 63.0f), mb = f16_bits(mmax / 63.0f);
        std::memcpy(out, &db, 2);
        std::memcpy(out + 2, &mb, 2);
        const float d = f16_value(db), dmin = f16_value(mb);
        uint8_t q[256];
        std::memset(q, 0, sizeof q);
        for (int j = 0; j < 8; j++) {  // quants from the scales as a decoder will read them back
            int sc, m;
            unpack_scale_min(packed, j, sc, m);
            const float step = d * (float)sc;
            if (step == 0.0f) continue;
            const float bias = dmin * (float)m;
            for (int i = 0; i < 32; i++) q[32 * j + i] = round_clamp_u8((row[32 * j + i] + bias) / step, 31.0f);
        }
        std::memset(out + 16, 0, 32);  // qh: byte l serves element l of every sub-block (q5_k.rs:27-33)
        for (int g = 0; g < 4; g++)
            for (int l = 0; l < 32; l++) {
                const uint8_t lo = q[64 * g + l], hi = q[64 * g + 32 + l];
                out[48 + 32 * g + l] = (uint8_t)((lo & 0xF) | ((hi & 0xF) << 4));
                out[16 + l] |= (uint8_t)(((lo >> 4) << (2 * g)) | ((hi >> 4) << (2 * g + 1)));
            }
    }
}

// Q6_K install encoder (crates/compute/src/quant_gguf/q6_k.rs:101-194): sub-block scale from the
// signed element of largest magnitude, int8 scales against the largest through a negative
// iscale, levels chosen against the f16-rounded d.
void encode_q6_k(const float* row, int64_t n, uint8_t* out) {
    for (int64_t sb = 0; sb < n / 256; sb++) {
        const float* x = row + sb * 256;
        uint8_t* blk = out + sb * 210;
        float sub_scale[16], biggest = 0.f;
        for (int j = 0; j < 16; j++) {
            float ext = 0.f;
            for (int i = 0; i < 16; i++)
                if (fabsf(x[16 * j + i]) > fabsf(ext)) ext = x[16 * j + i];
            sub_scale[j] = -ext / 32.0f;
            if (fabsf(sub_scale[j]) > fabsf(biggest)) biggest = sub_scale[j];
        }
        int8_t sc[16] = {0};
        _Float16 dh = (_Float16)0.0f;
        if (biggest != 0.f) {
            const float inv = -128.0f / biggest;
            for (int j = 0; j < 16; j++) sc[j] = (int8_t)std::min(std::max((int)roundf(inv * sub_scale[j]), -128), 127);
            dh = (_Float16)(1.0f / inv);
        }
        const float d = (float)dh;
        uint8_t lv[256];
        std::memset(lv, 32, sizeof lv);
        for (int j = 0; j < 16; j++) {
            const float step = d * (float)sc[j];
            if (step == 0.f) continue;
            for (int i = 0; i < 16; i++)
                lv[16 * j + i] = (uint8_t)((int)fminf(fmaxf(roundf(x[16 * j + i] / step), -32.f), 31.f) + 32);
        }
        for (int h = 0; h < 2; h++)
            for (int l = 0; l < 32; l++) {
                const uint8_t a = lv[128 * h + l], b = lv[128 * h + 32 + l], c = lv[128 * h + 64 + l], e = lv[128 * h + 96 + l];
                blk[64 * h + l] = (uint8_t)((a & 15) | ((c & 15) << 4));
                blk[64 * h + 32 + l] = (uint8_t)((b & 15) | ((e & 15) << 4));
                blk[128 + 32 * h + l] = (uint8_t)((a >> 4) | ((b >> 4) << 2) | ((c >> 4) << 4) | ((e >> 4) << 6));
            }
        std::memcpy(blk + 192, sc, 16);
        std::memcpy(blk + 208, &dh, 2);
    }
}

// MXFP4 install encoder.  The reference only decodes MXFP4 (quant_gguf_mxfp4.rs:114-141: value =
// kvalues[code] * 2^(e-128) with kvalues = 0,1,2,3,4,6,8,12 and their negatives); this encoder
// picks the smallest scale that keeps the block's largest magnitude within 12 * scale and then
// the nearest code for every element (first of equals; the second zero, code 8, is never used).
void encode_mxfp4(const float* row, int64_t n, uint8_t* out) {
    static const float kvalues[16] = {0.0f, 1.0f, 2.0f, 3.0f, 4.0f, 6.0f, 8.0f, 12.0f,
                                      0.0f, -1.0f, -2.0f, -3.0f, -4.0f, -6.0f, -8.0f, -12.0f};
    for (int64_t b = 0; b < n / 32; b++) {
        const float* block = row + b * 32;
        float amax = 0.0f;
        for (int k = 0; k < 32; k++) amax = std::fmax(amax, std::fabs(block[k]));
        int e = 2;
        if (amax > 0.0f) {
            int ex;
            (void)std::frexp(amax / 12.0f, &ex);
            e = std::min(std::max(ex + 128, 2), 254);
        }
        const uint32_t bits = (uint32_t)(e - 1) << 23;  // 2^(e-128)
        float d;
        std::memcpy(&d, &bits, 4);
        uint8_t* o = out + b * 17;
        o[0] = (uint8_t)e;
        uint8_t codes[32];
        for (int k = 0; k < 32; k++) {
            const float v = block[k] / d;
            int best = 0;
            float best_err = std::fabs(v - kvalues[0]);
            for (int c = 1; c < 16; c++) {
                if (c == 8) continue;
                const float err = std::fabs(v - kvalues[c]);
                if (err < best_err) {
                    best_err = err;
                    best = c;
                }
            }
            codes[k] = (uint8_t)best;
        }
        for (int j = 0; j < 16; j++) o[1 + j] = (uint8_t)(codes[j] | (codes[j + 16] << 4));
    }
}

int encode_row(int dtype, const float* src, int64_t cols, uint8_t* dst) {
    switch (dtype) {
        case TSV_F32: std::memcpy(dst, src, (size_t)cols * 4); return 0;
        case TSV_F16:
            for (int64_t i = 0; i < cols; i++) ((uint16_t*)dst)[i] = f16_bits(src[i]);
            return 0;
        case TSV_BF16:
            for (int64_t i = 0; i < cols; i++) ((uint16_t*)dst)[i] = bf16_bits(src[i]);
            return 0;
        case TSV_Q8_0: encode_q8_0(src, cols, dst); return 0;
        case TSV_Q4_K: encode_q4_k(src, cols, dst); return 0;
        case TSV_Q5_K: encode_q5_k(src, cols, dst); return 0;
        case TSV_Q6_K: encode_q6_k(src, cols, dst); return 0;
        case TSV_MXFP4: encode_mxfp4(src, cols, dst); return 0;
    }
    return -1;
}

inline uint64_t mix64(uint64_t x) {
    x += 0x9E3779B97F4A7C15ull;
    x = (x ^ (x >> 30)) * 0xBF58476D1CE4E5B9ull;
    x = (x ^ (x >> 27)) * 0x94D049BB133111EBull;
    return x ^ (x >> 31);
}

// Counter-based standard normals: pair p of a tensor is Box-Muller over two hashes of
// (seed, stream, p).  No state, so any row can be generated on any thread.
inline void normal_pair(uint64_t key, uint64_t p, double& z0, double& z1) {
    const uint64_t a = mix64(key ^ (2 * p * 0x9E3779B97F4A7C15ull));
    const uint64_t b = mix64(key ^ ((2 * p + 1) * 0x9E3779B97F4A7C15ull));
    const double u1 = ((double)(a >> 11) + 1.0) * (1.0 / 9007199254740992.0);  // (0, 1]
    const double u2 = (double)(b >> 11) * (1.0 / 9007199254740992.0);
    const double r = std::sqrt(-2.0 * std::log(u1)), t = 6.283185307179586476925 * u2;
    z0 = r * std::cos(t);
    z1 = r * std::sin(t);
}

template <class F>
void parallel_rows(int64_t rows, F f) {
    unsigned hw = std::thread::hardware_concurrency();
    int nt = (int)(hw ? (hw > 16 ? 16 : hw) : 4);
    if (rows < 2 * nt) nt = 1;
    if (nt == 1) {
        for (int64_t r = 0; r < rows; r++) f(r);
        return;
    }
    std::vector<std::thread> th;
    for (int t = 0; t < nt; t++)
        th.emplace_back([=] {
            for (int64_t r = t; r < rows; r += nt) f(r);
        });
    for (auto& x : th) x.join();
}

}  // namespace
}  // namespace tsv

extern "C" int64_t tsv_row_bytes(int32_t dtype, int64_t cols) { return tsv::row_bytes(dtype, cols); }

// crates/compute/src/rope.rs:296-372.  The two correction dimensions come from the wavelengths
// that fit beta_fast / beta_slow times into the original context; pairs below the first keep
// their frequency, pairs above the second are divided by the factor, linear mix between.
extern "C" int32_t tsv_yarn_frequencies(int32_t rotary_dim, float base, float factor, int64_t original_context,
                                        float beta_fast, float beta_slow, float* freqs, float* mscale) {
    if (rotary_dim < 2 || rotary_dim % 2 || !freqs || !mscale || !(base > 1.0f)) {
        tsv::set_error("yarn_frequencies: rotary_dim must be even and base > 1");
        return TSV_ERR_INVALID;
    }
    const bool on = factor > 0.0f;
    const float inv = on ? 1.0f / factor : 1.0f;
    auto corr = [&](float n_rot) {
        return (float)rotary_dim * logf((float)original_context / (n_rot * 2.0f * 3.14159265358979323846f)) /
               (2.0f * logf(base));
    };
    float lo = 0.0f, hi = 0.0f;
    if (on) {
        lo = fmaxf(floorf(corr(beta_fast)), 0.0f);
        hi = fminf(ceilf(corr(beta_slow)), (float)rotary_dim - 1.0f);
    }
    for (int p = 0; p < rotary_dim / 2; p++) {
        const float plain = powf(base, -((float)(2 * p)) / (float)rotary_dim);
        float f = plain;
        if (on) {
            const float y = ((float)p - lo) / fmaxf(hi - lo, 0.001f);
            const float keep = 1.0f - fminf(fmaxf(y, 0.0f), 1.0f);
            f = plain * (inv * (1.0f - keep) + keep);
        }
        freqs[p] = f;
    }
    *mscale = on ? 1.0f + 0.1f * logf(factor) : 1.0f;
    return TSV_OK;
}

extern "C" int32_t tsv_quantize_rows(int32_t dtype, const float* src, int64_t rows, int64_t cols, void* dst) {
    const int64_t rb = tsv::row_bytes(dtype, cols);
    if (rb < 0 || !src || !dst) {
        tsv::set_error("quantize: unsupported dtype or a column count that is not whole blocks");
        return TSV_ERR_INVALID;
    }
    tsv::parallel_rows(rows, [=](int64_t r) { tsv::encode_row(dtype, src + r * cols, cols, (uint8_t*)dst + r * rb); });
    return TSV_OK;
}

extern "C" int32_t tsv_synth_tensor(int32_t dtype, uint64_t seed, uint64_t stream, float sigma, int64_t rows,
                                    int64_t cols, void* dst) {
    const int64_t rb = tsv::row_bytes(dtype, cols);
    if (rb < 0 || !dst || (cols & 1)) {
        tsv::set_error("synth: unsupported dtype or column count");
        return TSV_ERR_INVALID;
    }
    const uint64_t key = tsv::mix64(seed ^ tsv::mix64(stream * 0xD1B54A32D192ED03ull + 1));
    tsv::parallel_rows(rows, [=](int64_t r) {
        std::vector<float> buf((size_t)cols);
        const uint64_t p0 = (uint64_t)r * (uint64_t)(cols / 2);
        for (int64_t c = 0; c < cols; c += 2) {
            double z0, z1;
            tsv::normal_pair(key, p0 + (uint64_t)(c / 2), z0, z1);
            buf[c] = (float)(z0 * (double)sigma);
            buf[c + 1] = (float)(z1 * (double)sigma);
        }
        tsv::encode_row(dtype, buf.data(), cols, (uint8_t*)dst + r * rb);
    });
    return TSV_OK;
}

extern "C" int32_t tsv_last_error(char* buf, int32_t cap) {
    const std::string& e = tsv::get_error();
    if (buf && cap > 0) {
        int32_t n = (int32_t)e.size() < cap - 1 ? (int32_t)e.size() : cap - 1;
        std::memcpy(buf, e.data(), (size_t)n);
        buf[n] = 0;
    }
    return (int32_t)e.size();
}
