// Block formats and scalar conversions of the CPU oracle (test infrastructure only).
// Follows crates/compute/src/quant_gguf/{q8_0,q4_k}.rs, quant_gguf_mxfp4.rs and quant.rs.
#include "tsoracle.h"

#include <cmath>
#include <cstring>
#include <vector>

#ifdef _OPENMP
#include <omp.h>
#endif

static inline uint32_t f32_bits(float x) {
    uint32_t u;
    std::memcpy(&u, &x, 4);
    return u;
}
static inline float bits_f32(uint32_t u) {
    float x;
    std::memcpy(&x, &u, 4);
    return x;
}

// IEEE binary32 -> binary16, round-to-nearest-even, what `half::f16::from_f32`
// computes (crates/core/src/primitives.rs:7-14 takes LogitValue = half::f16).
extern "C" uint16_t tso_f32_to_f16(float x) {
    uint32_t u = f32_bits(x);
    uint32_t sign = (u >> 16) & 0x8000u;
    uint32_t exp = (u >> 23) & 0xFFu;
    uint32_t man = u & 0x7FFFFFu;
    if (exp == 0xFF) {  // inf / nan
        if (man == 0) return (uint16_t)(sign | 0x7C00u);
        return (uint16_t)(sign | 0x7C00u | 0x0200u | (man >> 13));
    }
    int32_t e = (int32_t)exp - 127 + 15;
    if (e >= 0x1F) return (uint16_t)(sign | 0x7C00u);  // overflow -> inf
    if (e <= 0) {
        if (e < -10) return (uint16_t)sign;  // underflow to zero
        man |= 0x800000u;                   // make the leading one explicit
        uint32_t shift = (uint32_t)(14 - e);
        uint32_t half_man = man >> shift;
        uint32_t rem = man & ((1u << shift) - 1);
        uint32_t halfway = 1u << (shift - 1);
        if (rem > halfway || (rem == halfway && (half_man & 1))) half_man++;
        return (uint16_t)(sign | half_man);
    }
    uint32_t half = (uint32_t)(e << 10) | (man >> 13);
    uint32_t rem = man & 0x1FFFu;
    if (rem > 0x1000u || (rem == 0x1000u && (half & 1))) half++;  // may carry into exponent: correct
    return (uint16_t)(sign | half);
}

extern "C" float tso_f16_to_f32(uint16_t h) {
    uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0) {
        if (man == 0) return bits_f32(sign);
        // subnormal: normalise
        int e = -1;
        do {
            man <<= 1;
            e++;
        } while (!(man & 0x400u));
        man &= 0x3FFu;
        return bits_f32(sign | (uint32_t)(127 - 15 - e) << 23 | (man << 13));
    }
    if (exp == 0x1F) return bits_f32(sign | 0x7F800000u | (man << 13));
    return bits_f32(sign | ((exp + 127 - 15) << 23) | (man << 13));
}

// crates/compute/src/quant.rs:28-39
extern "C" uint16_t tso_f32_to_bf16(float x) {
    uint32_t bits = f32_bits(x);
    if (x != x) return (uint16_t)((bits >> 16) | 0x0040u);
    uint32_t lsb = (bits >> 16) & 1u;
    uint32_t bias = 0x7FFFu + lsb;
    return (uint16_t)((bits + bias) >> 16);
}
// crates/compute/src/quant.rs:14-17
extern "C" float tso_bf16_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

extern "C" int64_t tso_row_bytes(int dtype, int64_t n) {
    switch (dtype) {
        case TSO_F32: return n * 4;
        case TSO_F16:
        case TSO_BF16: return n * 2;
        case TSO_Q8_0: return n / 32 * 34;
        case TSO_Q4_K: return n / 256 * 144;
        case TSO_Q5_K: return n / 256 * 176;
        case TSO_Q6_K: return n / 256 * 210;
        case TSO_MXFP4: return (n + 31) / 32 * 17;
    }
    return -1;
}

static inline float clampf(float v, float lo, float hi) { return v < lo ? lo : (v > hi ? hi : v); }
// f32::min / f32::max on NaN-free inputs.  Rust leaves the sign of a +-0 tie unspecified;
// these keep the accumulator on a tie, so an all-zero block stores +0 scales (the two
// choices decode to the same values: x - (-0 * m) == x - (+0 * m)).
static inline float fold_min(float acc, float v) { return v < acc ? v : acc; }
static inline float fold_max(float acc, float v) { return v > acc ? v : acc; }

// Rust's f32::round is round-half-away-from-zero == C roundf.

// crates/compute/src/quant_gguf/q8_0.rs:56-77
extern "C" void tso_quantize_q8_0(const float* row, int64_t n, uint8_t* out) {
    for (int64_t b = 0; b < n / 32; b++) {
        const float* block = row + b * 32;
        float amax = 0.0f;
        for (int k = 0; k < 32; k++) amax = fold_max(amax, std::fabs(block[k]));
        uint16_t d = tso_f32_to_f16(amax / 127.0f);
        float d_f32 = tso_f16_to_f32(d);
        float inv = d_f32 == 0.0f ? 0.0f : 1.0f / d_f32;
        uint8_t* o = out + b * 34;
        o[0] = (uint8_t)(d & 0xFF);
        o[1] = (uint8_t)(d >> 8);
        for (int k = 0; k < 32; k++) {
            float r = roundf(block[k] * inv);
            int32_t q = (int32_t)r;  // finite by construction
            if (q < -127) q = -127;
            if (q > 127) q = 127;
            o[2 + k] = (uint8_t)(int8_t)q;
        }
    }
}

// crates/compute/src/quant_gguf/q8_0.rs:19-47
extern "C" void tso_dequantize_q8_0(const uint8_t* blocks, int64_t n, float* out) {
    for (int64_t b = 0; b < n / 32; b++) {
        const uint8_t* p = blocks + b * 34;
        float d = tso_f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
        for (int k = 0; k < 32; k++) out[b * 32 + k] = (float)(int8_t)p[2 + k] * d;
    }
}

// crates/compute/src/quant_gguf/q4_k.rs:43-54
extern "C" void tso_q4_k_scale_min(int j, const uint8_t* packed, uint8_t* sc, uint8_t* mn) {
    if (j < 4) {
        *sc = packed[j] & 63;
        *mn = packed[j + 4] & 63;
    } else {
        *sc = (uint8_t)((packed[j + 4] & 0xF) | ((packed[j - 4] >> 6) << 4));
        *mn = (uint8_t)((packed[j + 4] >> 4) | ((packed[j] >> 6) << 4));
    }
}

// crates/compute/src/quant_gguf/q4_k.rs:67-108
extern "C" void tso_dequantize_q4_k(const uint8_t* blocks, int64_t n, float* out) {
    for (int64_t b = 0; b < n / 256; b++) {
        const uint8_t* p = blocks + b * 144;
        float d = tso_f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
        float dmin = tso_f16_to_f32((uint16_t)(p[2] | (p[3] << 8)));
        const uint8_t* packed = p + 4;
        const uint8_t* qs = p + 16;
        for (int g = 0; g < 4; g++) {
            uint8_t sc_lo, m_lo, sc_hi, m_hi;
            tso_q4_k_scale_min(2 * g, packed, &sc_lo, &m_lo);
            tso_q4_k_scale_min(2 * g + 1, packed, &sc_hi, &m_hi);
            float d_lo = d * (float)sc_lo, min_lo = dmin * (float)m_lo;
            float d_hi = d * (float)sc_hi, min_hi = dmin * (float)m_hi;
            const uint8_t* group = qs + g * 32;
            float* at = out + b * 256 + g * 64;
            for (int l = 0; l < 32; l++) {
                uint8_t byte = group[l];
                at[l] = d_lo * (float)(byte & 0xF) - min_lo;
                at[32 + l] = d_hi * (float)(byte >> 4) - min_hi;
            }
        }
    }
}

// crates/compute/src/quant_gguf/q4_k.rs:126-204
extern "C" void tso_quantize_q4_k(const float* row, int64_t n, uint8_t* out) {
    for (int64_t b = 0; b < n / 256; b++) {
        const float* block = row + b * 256;
        float scales[8], mins[8];
        for (int j = 0; j < 8; j++) {
            const float* sub = block + j * 32;
            float lo = 0.0f;
            for (int i = 0; i < 32; i++) lo = fold_min(lo, sub[i]);
            float hi = lo;
            for (int i = 0; i < 32; i++) hi = fold_max(hi, sub[i]);
            scales[j] = (hi - lo) / 15.0f;
            mins[j] = -lo;
        }
        float max_scale = 0.0f, max_min = 0.0f;
        for (int j = 0; j < 8; j++) {
            max_scale = fold_max(max_scale, scales[j]);
            max_min = fold_max(max_min, mins[j]);
        }
        float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
        float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
        uint8_t packed[12] = {0};
        for (int j = 0; j < 8; j++) {
            uint8_t ls = (uint8_t)clampf(roundf(scales[j] * inv_scale), 0.0f, 63.0f);
            uint8_t lm = (uint8_t)clampf(roundf(mins[j] * inv_min), 0.0f, 63.0f);
            if (j < 4) {
                packed[j] |= ls;
                packed[j + 4] |= lm;
            } else {
                packed[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                packed[j - 4] |= (uint8_t)((ls >> 4) << 6);
                packed[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        uint16_t d = tso_f32_to_f16(max_scale / 63.0f);
        uint16_t dmin = tso_f32_to_f16(max_min / 63.0f);
        float d_f = tso_f16_to_f32(d), dmin_f = tso_f16_to_f32(dmin);
        uint8_t quants[256] = {0};
        for (int j = 0; j < 8; j++) {
            uint8_t sc, m;
            tso_q4_k_scale_min(j, packed, &sc, &m);
            float step = d_f * (float)sc;
            if (step == 0.0f) continue;
            float bias = dmin_f * (float)m;
            for (int i = 0; i < 32; i++) {
                float w = block[j * 32 + i];
                quants[j * 32 + i] = (uint8_t)clampf(roundf((w + bias) / step), 0.0f, 15.0f);
            }
        }
        uint8_t* o = out + b * 144;
        o[0] = (uint8_t)(d & 0xFF);
        o[1] = (uint8_t)(d >> 8);
        o[2] = (uint8_t)(dmin & 0xFF);
        o[3] = (uint8_t)(dmin >> 8);
        std::memcpy(o + 4, packed, 12);
        for (int g = 0; g < 4; g++)
            for (int l = 0; l < 32; l++)
                o[16 + g * 32 + l] = (uint8_t)(quants[g * 64 + l] | (quants[g * 64 + 32 + l] << 4));
    }
}

// crates/compute/src/quant_gguf/q5_k.rs:47-96.  Q4_K plus a fifth bit per element: d, dmin, the same
// 12 packed 6-bit scales / mins, then 32 bytes `qh` and 128 nibble bytes.  Byte qh[l] serves the
// elements l, l + 32, l + 64, ... of the superblock; group g (64 elements) reads bit 2g for its low
// nibbles and bit 2g + 1 for its high ones.
extern "C" void tso_dequantize_q5_k(const uint8_t* blocks, int64_t n, float* out) {
    for (int64_t b = 0; b < n / 256; b++) {
        const uint8_t* p = blocks + b * 176;
        float d = tso_f16_to_f32((uint16_t)(p[0] | (p[1] << 8)));
        float dmin = tso_f16_to_f32((uint16_t)(p[2] | (p[3] << 8)));
        const uint8_t* packed = p + 4;
        const uint8_t* qh = p + 16;
        const uint8_t* ql = p + 48;
        for (int g = 0; g < 4; g++) {
            uint8_t sc_lo, m_lo, sc_hi, m_hi;
            tso_q4_k_scale_min(2 * g, packed, &sc_lo, &m_lo);
            tso_q4_k_scale_min(2 * g + 1, packed, &sc_hi, &m_hi);
            float d_lo = d * (float)sc_lo, min_lo = dmin * (float)m_lo;
            float d_hi = d * (float)sc_hi, min_hi = dmin * (float)m_hi;
            const uint8_t* group = ql + g * 32;
            float* at = out + b * 256 + g * 64;
            for (int l = 0; l < 32; l++) {
                uint8_t byte = group[l], hb = qh[l];
                uint8_t q_lo = (uint8_t)((byte & 0xF) + (((hb >> (2 * g)) & 1) << 4));
                uint8_t q_hi = (uint8_t)((byte >> 4) + (((hb >> (2 * g + 1)) & 1) << 4));
                at[l] = d_lo * (float)q_lo - min_lo;
                at[32 + l] = d_hi * (float)q_hi - min_hi;
            }
        }
    }
}

// NOT IN THE REFERENCE (it only decodes Q5_K): the Q4_K min/max fitter of q4_k.rs:126-204 with 31
// levels per sub-block instead of 15, so that synthetic weights can be stored in this format.
extern "C" void tso_quantize_q5_k(const float* row, int64_t n, uint8_t* out) {
    for (int64_t b = 0; b < n / 256; b++) {
        const float* block = row + b * 256;
        float scales[8], mins[8];
        for (int j = 0; j < 8; j++) {
            const float* sub = block + j * 32;
            float lo = 0.0f;
            for (int i = 0; i < 32; i++) lo = fold_min(lo, sub[i]);
            float hi = lo;
            for (int i = 0; i < 32; i++) hi = fold_max(hi, sub[i]);
            scales[j] = (hi - lo) / 31.0f;
            mins[j] = -lo;
        }
        float max_scale = 0.0f, max_min = 0.0f;
        for (int j = 0; j < 8; j++) {
            max_scale = fold_max(max_scale, scales[j]);
            max_min = fold_max(max_min, mins[j]);
        }
        float inv_scale = max_scale > 0.0f ? 63.0f / max_scale : 0.0f;
        float inv_min = max_min > 0.0f ? 63.0f / max_min : 0.0f;
        uint8_t packed[12] = {0};
        for (int j = 0; j < 8; j++) {
            uint8_t ls = (uint8_t)clampf(roundf(scales[j] * inv_scale), 0.0f, 63.0f);
            uint8_t lm = (uint8_t)clampf(roundf(mins[j] * inv_min), 0.0f, 63.0f);
            if (j < 4) {
                packed[j] |= ls;
                packed[j + 4] |= lm;
            } else {
                packed[j + 4] = (uint8_t)((ls & 0xF) | ((lm & 0xF) << 4));
                packed[j - 4] |= (uint8_t)((ls >> 4) << 6);
                packed[j] |= (uint8_t)((lm >> 4) << 6);
            }
        }
        uint16_t d = tso_f32_to_f16(max_scale / 63.0f);
        uint16_t dmin = tso_f32_to_f16(max_min / 63.0f);
        float d_f = tso_f16_to_f32(d), dmin_f = tso_f16_to_f32(dmin);
        uint8_t quants[256] = {0};
        for (int j = 0; j < 8; j++) {
            uint8_t sc, m;
            tso_q4_k_scale_min(j, packed, &sc, &m);
            float step = d_f * (float)sc;
            if (step == 0.0f) continue;
            float bias = dmin_f * (float)m;
            for (int i = 0; i < 32; i++)
                quants[j * 32 + i] = (uint8_t)clampf(roundf((block[j * 32 + i] + bias) / step), 0.0f, 31.0f);
        }
        uint8_t* o = out + b * 176;
        std::memset(o, 0, 176);
        o[0] = (uint8_t)(d & 0xFF);
        o[1] = (uint8_t)(d >> 8);
        o[2] = (uint8_t)(dmin & 0xFF);
        o[3] = (uint8_t)(dmin >> 8);
        std::memcpy(o + 4, packed, 12);
        for (int g = 0; g < 4; g++)
            for (int l = 0; l < 32; l++) {
                const uint8_t q_lo = quants[g * 64 + l], q_hi = quants[g * 64 + 32 + l];
                o[48 + g * 32 + l] = (uint8_t)((q_lo & 0xF) | ((q_hi & 0xF) << 4));
                o[16 + l] |= (uint8_t)(((q_lo >> 4) << (2 * g)) | ((q_hi >> 4) << (2 * g + 1)));
            }
    }
}

// crates/compute/src/quant_gguf_mxfp4.rs:76-78
static const float MXFP4_VALUES[16] = {0.0f, 1.0f, 2.0f,  3.0f,  4.0f,  6.0f,  8.0f,  12.0f,
                                       0.0f, -1.0f, -2.0f, -3.0f, -4.0f, -6.0f, -8.0f, -12.0f};

// crates/compute/src/quant_gguf_mxfp4.rs:95-102
extern "C" float tso_mxfp4_scale(uint8_t e) {
    uint32_t bits = e < 2 ? (0x00200000u << e) : ((uint32_t)(e - 1) << 23);
    return bits_f32(bits);
}

// crates/compute/src/quant_gguf_mxfp4.rs:114-141
extern "C" void tso_dequantize_mxfp4(const uint8_t* blocks, int64_t n, float* out) {
    int64_t block_count = (n + 31) / 32;
    for (int64_t b = 0; b < block_count; b++) {
        const uint8_t* p = blocks + b * 17;
        float d = tso_mxfp4_scale(p[0]);
        for (int j = 0; j < 16; j++) {
            int64_t lo = b * 32 + j, hi = lo + 16;
            if (lo < n) out[lo] = MXFP4_VALUES[p[1 + j] & 0x0F] * d;
            if (hi < n) out[hi] = MXFP4_VALUES[p[1 + j] >> 4] * d;
        }
    }
}

// No counterpart in the reference (quant_gguf_mxfp4.rs:40-48 says it has no encoder).
// Shared exponent: the smallest e whose largest code (12 * 2^(e-128)) covers amax;
// then each element takes the nearest codebook value, ties to the lower index.
extern "C" void tso_quantize_mxfp4(const float* row, int64_t n, uint8_t* out) {
    for (int64_t b = 0; b < n / 32; b++) {
        const float* block = row + b * 32;
        float amax = 0.0f;
        for (int k = 0; k < 32; k++) amax = std::fmax(amax, std::fabs(block[k]));
        int e = 2;
        if (amax > 0.0f) {
            int ex;
            std::frexp(amax / 12.0f, &ex);  // amax/12 = f * 2^ex, f in [0.5,1)
            e = ex + 128;                   // 2^(e-128) >= amax/12
            if (e < 2) e = 2;
            if (e > 254) e = 254;
        }
        float d = tso_mxfp4_scale((uint8_t)e);
        uint8_t* o = out + b * 17;
        o[0] = (uint8_t)e;
        uint8_t codes[32];
        for (int k = 0; k < 32; k++) {
            float v = block[k] / d;
            int best = 0;
            float best_err = std::fabs(v - MXFP4_VALUES[0]);
            for (int c = 1; c < 16; c++) {
                if (c == 8) continue;  // the second zero is never emitted
                float err = std::fabs(v - MXFP4_VALUES[c]);
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

extern "C" void tso_dequantize_row(int dtype, const uint8_t* row, int64_t n, float* out) {
    switch (dtype) {
        case TSO_F32: std::memcpy(out, row, (size_t)n * 4); break;
        case TSO_F16:
            for (int64_t i = 0; i < n; i++) out[i] = tso_f16_to_f32(((const uint16_t*)row)[i]);
            break;
        case TSO_BF16:
            for (int64_t i = 0; i < n; i++) out[i] = tso_bf16_to_f32(((const uint16_t*)row)[i]);
            break;
        case TSO_Q8_0: tso_dequantize_q8_0(row, n, out); break;
        case TSO_Q4_K: tso_dequantize_q4_k(row, n, out); break;
        case TSO_Q5_K: tso_dequantize_q5_k(row, n, out); break;
        case TSO_Q6_K: tso_dequantize_q6_k(row, n, out); break;
        case TSO_MXFP4: tso_dequantize_mxfp4(row, n, out); break;
    }
}

// crates/compute/src/quant_gguf/q6_k.rs:44-88.  A superblock is two halves of 128 elements; in a
// half, byte l of `ql` (and l + 32) and byte l of `qh` serve the four elements l, l + 32, l + 64,
// l + 96, each with its own scale (is, is + 2, is + 4, is + 6); stored levels carry a bias of 32.
extern "C" void tso_dequantize_q6_k(const uint8_t* blocks, int64_t n, float* out) {
    for (int64_t b = 0; b < n / 256; b++) {
        const uint8_t* blk = blocks + b * 210;
        uint16_t db;
        std::memcpy(&db, blk + 208, 2);
        const float d = tso_f16_to_f32(db);
        for (int h = 0; h < 2; h++) {
            const uint8_t* ql = blk + h * 64;
            const uint8_t* qh = blk + 128 + h * 32;
            const int8_t* sc = (const int8_t*)blk + 192 + h * 8;
            float* o = out + b * 256 + h * 128;
            for (int l = 0; l < 32; l++) {
                const int is = l / 16;
                const int q[4] = {(int)((ql[l] & 0xF) | ((qh[l] & 3) << 4)) - 32,
                                  (int)((ql[l + 32] & 0xF) | (((qh[l] >> 2) & 3) << 4)) - 32,
                                  (int)((ql[l] >> 4) | (((qh[l] >> 4) & 3) << 4)) - 32,
                                  (int)((ql[l + 32] >> 4) | (((qh[l] >> 6) & 3) << 4)) - 32};
                for (int k = 0; k < 4; k++) o[l + k * 32] = d * (float)sc[is + k * 2] * (float)q[k];
            }
        }
    }
}

// crates/compute/src/quant_gguf/q6_k.rs:101-194: per 16-element sub-block the signed element of
// largest magnitude sets the scale (-extreme / 32), the scales are quantised to int8 against the
// largest one through a negative iscale, d is rounded through f16 before the levels are chosen.
extern "C" void tso_quantize_q6_k(const float* row, int64_t n, uint8_t* out) {
    for (int64_t b = 0; b < n / 256; b++) {
        const float* block = row + b * 256;
        uint8_t* blk = out + b * 210;
        float scales[16], max_scale = 0.0f;
        for (int j = 0; j < 16; j++) {
            float extreme = 0.0f;
            for (int i = 0; i < 16; i++)
                if (std::fabs(block[j * 16 + i]) > std::fabs(extreme)) extreme = block[j * 16 + i];
            scales[j] = -extreme / 32.0f;
            if (std::fabs(scales[j]) > std::fabs(max_scale)) max_scale = scales[j];
        }
        int8_t sc[16] = {0};
        uint16_t dbits = tso_f32_to_f16(0.0f);
        if (max_scale != 0.0f) {
            const float iscale = -128.0f / max_scale;
            for (int j = 0; j < 16; j++) {
                int v = (int)std::round(iscale * scales[j]);  // f32::round: half away from zero
                sc[j] = (int8_t)std::min(std::max(v, -128), 127);
            }
            dbits = tso_f32_to_f16(1.0f / iscale);
        }
        const float d = tso_f16_to_f32(dbits);
        uint8_t levels[256];
        std::memset(levels, 32, sizeof levels);
        for (int j = 0; j < 16; j++) {
            const float step = d * (float)sc[j];
            if (step == 0.0f) continue;
            for (int i = 0; i < 16; i++) {
                float q = std::round(block[j * 16 + i] / step);
                q = std::min(std::max(q, -32.0f), 31.0f);
                levels[j * 16 + i] = (uint8_t)((int)q + 32);
            }
        }
        std::memset(blk, 0, 210);
        for (int h = 0; h < 2; h++)
            for (int l = 0; l < 32; l++) {
                const uint8_t* v = levels + h * 128 + l;
                blk[h * 64 + l] = (uint8_t)((v[0] & 0xF) | ((v[64] & 0xF) << 4));
                blk[h * 64 + l + 32] = (uint8_t)((v[32] & 0xF) | ((v[96] & 0xF) << 4));
                blk[128 + h * 32 + l] =
                    (uint8_t)((v[0] >> 4) | ((v[32] >> 4) << 2) | ((v[64] >> 4) << 4) | ((v[96] >> 4) << 6));
            }
        std::memcpy(blk + 192, sc, 16);
        std::memcpy(blk + 208, &dbits, 2);
    }
}

// dequant_q4_k_gemv / dequant_q8_0_gemv (q4_k.rs:207-220, q8_0.rs:80-93): dequantize the
// row to fp32, multiply elementwise, sum sequentially in index order.
extern "C" void tso_gemv(int dtype, const uint8_t* w, int64_t rows, int64_t cols, const float* x,
                         float* y) {
    int64_t rb = tso_row_bytes(dtype, cols);
    std::vector<float> deq((size_t)cols);
    for (int64_t r = 0; r < rows; r++) {
        tso_dequantize_row(dtype, w + r * rb, cols, deq.data());
        float acc = 0.0f;
        for (int64_t k = 0; k < cols; k++) acc += deq[k] * x[k];
        y[r] = acc;
    }
}
