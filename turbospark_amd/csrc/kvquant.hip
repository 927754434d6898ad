// TurboQuant KV rows: the codec's tables (host) and the kernel that runs before the attention of a
// quantized layer.
//
// A quantized layer keeps, per position and kv head, one f32 norm and the packed codebook indices of
// the row's rotated unit vector (crates/compute/src/kv_quant.rs:340-382; the row layout of
// crates/gpu/tests/kv_quantize_parity.rs:22-38: [norm][words]).  Attention runs in the rotated space
// (crates/compute/src/kv_quant_attention.rs:58-136): q is rotated once with the key signs, scores are
// <q_rot, codebook[idx]> * norm, the values are summed as norm * codebook[idx] and the sum is rotated
// back once with the value signs.  Here the rows norm * codebook[idx] are written, as fp16, into an
// fp16 cache of one layer's size that all quantized layers share, and the ordinary attention kernels
// read that; the merge kernel rotates the result back.
//
// The pass's own rows arrive in that shared cache as fp16 (the staging row of
// crates/runtime/src/kv_write.rs:66-118) and are quantized from there: norm as the f32 sum of squares
// in index order, unit = x * (1 / max(norm, 1e-6)), the butterflies of crates/compute/src/wht.rs:15-29
// in their order with each stage scaled by 1/sqrt(2), one index per coordinate as the count of
// midpoints below it, bits LSB first.  Every operation is a single rounded f32 operation in the
// reference's order, so the words and the norm are the reference's by bits.
#include <algorithm>
#include <cmath>
#include <vector>

#include "tsv_internal.h"

namespace tsv {

// ---------------------------------------------------------------- tables (host)

// crates/compute/src/kv_quant.rs:54-81
void tq_sign_vector(int dim, uint64_t seed, float* out) {
    uint64_t state = seed + (uint64_t)dim * 7919ull;
    for (int i = 0; i < dim; i++) {
        state += 0x9E3779B97F4A7C15ull;
        uint64_t z = state;
        z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
        z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
        z ^= z >> 31;
        out[i] = (z & 1ull) ? 1.0f : -1.0f;
    }
}

// crates/compute/src/kv_quant.rs:166-256: Lloyd-Max centroids of the density (1 - x^2)^((dim - 3) / 2)
// on 32768 grid points, at most 100 iterations, all in f64.  The grid is sorted and so are the
// boundaries, so one walk over the grid serves every level: each level's sums take its points in
// ascending order, as the reference's scan per level does.
std::vector<float> tq_codebook(int dim, int bits) {
    const int levels = 1 << bits, G = 32768;
    std::vector<double> grid(G), w(G), cdf(G);
    for (int i = 0; i < G; i++) grid[i] = (-1.0 + 1e-6) + ((double)i / ((double)G - 1.0)) * (2.0 - 2e-6);
    double top = -INFINITY;
    for (int i = 0; i < G; i++) {
        w[i] = (((double)dim - 3.0) / 2.0) * std::log(std::max(1.0 - grid[i] * grid[i], 1e-30));
        top = std::max(top, w[i]);
    }
    double total = 0.0;
    for (int i = 0; i < G; i++) total += (w[i] = std::exp(w[i] - top));
    for (int i = 0; i < G; i++) w[i] = total > 0.0 ? w[i] / total : 1.0 / (double)G;
    double run = 0.0;
    for (int i = 0; i < G; i++) cdf[i] = (run += w[i]);
    std::vector<double> c(levels);
    for (int l = 0; l < levels; l++) {  // the quantile (l + 0.5) / levels, by linear interpolation of the cdf
        const double q = ((double)l + 0.5) / (double)levels;
        if (q <= cdf.front()) {
            c[l] = grid.front();
        } else if (q >= cdf.back()) {
            c[l] = grid.back();
        } else {
            const size_t i = (size_t)(std::lower_bound(cdf.begin(), cdf.end(), q) - cdf.begin());
            if (cdf[i] == q || cdf[i] == cdf[i - 1])
                c[l] = cdf[i] == q ? grid[i] : grid[i - 1];
            else
                c[l] = grid[i - 1] + (grid[i] - grid[i - 1]) * (q - cdf[i - 1]) / (cdf[i] - cdf[i - 1]);
        }
    }
    for (int it = 0; it < 100; it++) {
        std::vector<double> edge(levels + 1);
        edge[0] = -1.0;
        edge[levels] = 1.0;
        for (int l = 1; l < levels; l++) edge[l] = 0.5 * (c[l - 1] + c[l]);
        std::vector<double> num(levels, 0.0), den(levels, 0.0);
        int l = 0;
        for (int g = 0; g < G; g++) {
            const double x = grid[g];
            if (x < edge[0]) continue;
            while (l + 1 < levels && !(x < edge[l + 1])) l++;  // level l holds [edge l, edge l+1), the last one its right end too
            if (x > edge[levels]) break;
            num[l] += w[g] * x;
            den[l] += w[g];
        }
        double moved = 0.0;
        for (int i = 0; i < levels; i++) {
            const double nx = den[i] > 0.0 ? num[i] / den[i] : c[i];
            moved = std::max(moved, std::fabs(c[i] - nx));
            c[i] = nx;
        }
        if (moved < 1e-6) break;
    }
    std::vector<float> out(levels);
    for (int i = 0; i < levels; i++) out[i] = (float)c[i];
    return out;
}

int tq_words(int hd, int bits) { return (hd * bits + 31) / 32; }

// signs, codebook and midpoints of one side (key: seed 0, value: seed 1; kv_quant.rs:33-36) in one
// device allocation of TQ_TABLE_FLOATS floats
int tq_upload_side(int hd, int bits, uint64_t seed, float* dev, TqSide* out) {
    std::vector<float> host(TQ_TABLE_FLOATS, 0.f);
    tq_sign_vector(hd, seed, host.data());
    const std::vector<float> cb = tq_codebook(hd, bits);
    std::copy(cb.begin(), cb.end(), host.begin() + 512);
    for (size_t i = 0; i + 1 < cb.size(); i++) host[512 + 16 + i] = 0.5f * (cb[i] + cb[i + 1]);  // kv_quant.rs:262-264
    TSV_HIP(hipMemcpy(dev, host.data(), host.size() * 4, hipMemcpyHostToDevice));
    out->signs = dev;
    out->cb = dev + 512;
    out->mid = dev + 512 + 16;
    out->bits = bits;
    out->words = tq_words(hd, bits);
    return TSV_OK;
}

// ---------------------------------------------------------------- the kernel

namespace {

__device__ __forceinline__ void lds_order() {
    // one wave writes and reads its own LDS rows: program order is all the hardware needs, the
    // fence keeps the compiler to it
    __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
    __builtin_amdgcn_wave_barrier();
}

// crates/compute/src/wht.rs:15-29, bottom-up: stage h pairs i with i + h, (lo + hi) and (lo - hi), each
// scaled by 1/sqrt(2).  Lane l holds elements l and l + 64.
template <int EPL>
__device__ __forceinline__ void wht(float (&e)[EPL], int lane, float c) {
#pragma unroll
    for (int h = 1; h < 64; h <<= 1) {
#pragma unroll
        for (int j = 0; j < EPL; j++) {
            const float other = __shfl_xor(e[j], h);
            e[j] = __fmul_rn((lane & h) ? __fsub_rn(other, e[j]) : __fadd_rn(e[j], other), c);
        }
    }
    if (EPL == 2) {
        const float lo = e[0], hi = e[EPL - 1];
        e[0] = __fmul_rn(__fadd_rn(lo, hi), c);
        e[EPL - 1] = __fmul_rn(__fsub_rn(lo, hi), c);
    }
}

__device__ __forceinline__ long k_at(const TqArgs& a, int head, int pos, int d) { return ((long)head * a.cap + pos) * a.hd + d; }
__device__ __forceinline__ long v_at(const TqArgs& a, int head, int pos, int d) {
    const int po = pos & 15;
    return ((long)head * (a.cap >> 4) + (pos >> 4)) * (a.hd * 16) + (((d >> 4) * 64) + (po >> 2) * 16 + (d & 15)) * 4 + (po & 3);
}

__device__ __forceinline__ uint32_t index_at(const uint32_t* words, int i, int bits) {
    const uint32_t bit = (uint32_t)i * (uint32_t)bits, w = bit >> 5, off = bit & 31;
    uint32_t v = words[w] >> off;
    if (off + bits > 32) v |= words[w + 1] << (32 - off);
    return v & ((1u << bits) - 1u);
}

// what a stored row reads as in the rotated space: fp16(norm * codebook[idx]), one rounded product
__device__ __forceinline__ _Float16 decoded(float norm, float level) {
    float p = __fmul_rn(norm, level);
    asm volatile("" : "+v"(p));  // the product is rounded to f32 before it is rounded to fp16
    return (_Float16)p;
}

// q row (b, qh): rotate with the key signs, in place
template <int HD>
__device__ void rotate_q(const TqArgs& a, int b, int qh, int lane) {
    constexpr int EPL = HD / 64;
    _Float16* row = (_Float16*)a.q16 + ((long)b * a.nq + qh) * HD;
    float e[EPL];
#pragma unroll
    for (int j = 0; j < EPL; j++) e[j] = __fmul_rn((float)row[lane + 64 * j], a.k.signs[lane + 64 * j]);
    wht<EPL>(e, lane, a.inv_sqrt2);
#pragma unroll
    for (int j = 0; j < EPL; j++) row[lane + 64 * j] = (_Float16)e[j];
}

// the pass's row at `pos`, kv head `head`: fp16 row in the shared cache -> norm + words in the layer's
// store, and the decoded row back into the shared cache
template <int HD>
__device__ void commit_row(const TqArgs& a, bool value, int pos, int head, int lane, float* s_row, uint32_t* s_words) {
    constexpr int EPL = HD / 64;
    const TqSide& t = value ? a.v : a.k;
    _Float16* cache = (_Float16*)(value ? a.vc : a.kc);
    float x[EPL];
#pragma unroll
    for (int j = 0; j < EPL; j++) {
        const int d = lane + 64 * j;
        x[j] = (float)cache[value ? v_at(a, head, pos, d) : k_at(a, head, pos, d)];
        s_row[d] = x[j];
    }
    if (lane < t.words + 1) s_words[lane] = 0;
    lds_order();
    float ss = 0.f;
    for (int i = 0; i < HD; i++) ss = __fadd_rn(ss, __fmul_rn(s_row[i], s_row[i]));
    const float norm = sqrtf(ss);  // correctly rounded, as is the division (the toolchain's default for f32)
    const float inv = 1.0f / fmaxf(norm, 1e-6f);
    float e[EPL];
#pragma unroll
    for (int j = 0; j < EPL; j++) e[j] = __fmul_rn(__fmul_rn(x[j], inv), t.signs[lane + 64 * j]);
    wht<EPL>(e, lane, a.inv_sqrt2);
    const int n_mid = (1 << t.bits) - 1;
    uint32_t idx[EPL];
#pragma unroll
    for (int j = 0; j < EPL; j++) {
        uint32_t c = 0;
        for (int i = 0; i < n_mid; i++) c += e[j] > t.mid[i] ? 1u : 0u;
        idx[j] = c;
        const uint32_t bit = (uint32_t)(lane + 64 * j) * (uint32_t)t.bits, w = bit >> 5, off = bit & 31;
        atomicOr(&s_words[w], c << off);
        if (off + t.bits > 32) atomicOr(&s_words[w + 1], c >> (32 - off));
    }
    lds_order();
    uint32_t* out = (value ? a.vq : a.kq) + ((long)pos * a.nkv + head) * (1 + t.words);
    if (lane == 0) out[0] = __builtin_bit_cast(uint32_t, norm);
    if (lane < t.words) out[1 + lane] = s_words[lane];
#pragma unroll
    for (int j = 0; j < EPL; j++) {
        const int d = lane + 64 * j;
        cache[value ? v_at(a, head, pos, d) : k_at(a, head, pos, d)] = decoded(norm, t.cb[idx[j]]);
    }
    lds_order();
}

// a stored key row back into the shared cache
template <int HD>
__device__ void expand_k(const TqArgs& a, int pos, int head, int lane) {
    constexpr int EPL = HD / 64;
    const uint32_t* row = a.kq + ((long)pos * a.nkv + head) * (1 + a.k.words);
    const float norm = __builtin_bit_cast(float, row[0]);
    _Float16 h[EPL];
#pragma unroll
    for (int j = 0; j < EPL; j++) h[j] = decoded(norm, a.k.cb[index_at(row + 1, EPL * lane + j, a.k.bits)]);
    _Float16* dst = (_Float16*)a.kc + k_at(a, head, pos, EPL * lane);
    if (EPL == 2) {
        *(uint32_t*)dst = (uint32_t)__builtin_bit_cast(uint16_t, h[0]) | ((uint32_t)__builtin_bit_cast(uint16_t, h[EPL - 1]) << 16);
    } else {
        dst[0] = h[0];
    }
}

// sixteen stored value rows back into the shared cache: lane (j, dl) holds positions 4j .. 4j+3 of
// dimension 16 dh + dl, eight contiguous bytes of the block's layout
template <int HD>
__device__ void expand_v(const TqArgs& a, int blk, int head, int base, int lane) {
    const int j = lane >> 4, dl = lane & 15, p0 = blk * 16 + 4 * j;
    const uint32_t* rows[4];
    float norm[4];
#pragma unroll
    for (int i = 0; i < 4; i++) {
        rows[i] = a.vq + ((long)min(p0 + i, base - 1) * a.nkv + head) * (1 + a.v.words);
        norm[i] = __builtin_bit_cast(float, rows[i][0]);
    }
    _Float16* dst = (_Float16*)a.vc + ((long)head * (a.cap >> 4) + blk) * (HD * 16);
    const bool whole = p0 + 4 <= base;
#pragma unroll 2
    for (int dh = 0; dh < HD / 16; dh++) {
        const int d = dh * 16 + dl;
        uint16_t h[4];
#pragma unroll
        for (int i = 0; i < 4; i++) h[i] = __builtin_bit_cast(uint16_t, decoded(norm[i], a.v.cb[index_at(rows[i] + 1, d, a.v.bits)]));
        _Float16* at = dst + (dh * 64 + lane) * 4;
        if (whole) {
            *(uint2*)at = uint2{(uint32_t)h[0] | ((uint32_t)h[1] << 16), (uint32_t)h[2] | ((uint32_t)h[3] << 16)};
        } else {  // the block the pass's own rows start in: those are the other kernel section's to write
#pragma unroll
            for (int i = 0; i < 4; i++)
                if (p0 + i < base) at[i] = __builtin_bit_cast(_Float16, h[i]);
        }
    }
}

// One wave per unit of work, units in four classes: q rows to rotate, the pass's K and V rows to
// quantize, stored K rows and stored blocks of sixteen V rows to decode.  The classes touch disjoint
// bytes, so their order does not matter.
template <int HD>
__global__ __launch_bounds__(256) void k_tq_prepare(TqArgs a) {
    __shared__ float s_row[4][HD];
    __shared__ uint32_t s_words[4][HD / 2 + 1];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = a.m_hint, base = a.base_hint >= 0 ? a.base_hint : a.vp->base;
    const long n_q = (long)m * a.nq, n_commit = 2l * m * a.nkv, n_k = (long)base * a.nkv, n_v = (long)((base + 15) >> 4) * a.nkv;
    const long total = n_q + n_commit + n_k + n_v;
    for (long u = (long)blockIdx.x * 4 + wave; u < total; u += (long)gridDim.x * 4) {
        if (u < n_q) {
            rotate_q<HD>(a, (int)(u / a.nq), (int)(u % a.nq), lane);
        } else if (u < n_q + n_commit) {
            const long r = u - n_q;
            const bool value = r >= (long)m * a.nkv;
            const int rr = (int)(value ? r - (long)m * a.nkv : r);
            commit_row<HD>(a, value, (base + rr / a.nkv) % a.cap, rr % a.nkv, lane, s_row[wave], s_words[wave]);
        } else if (u < n_q + n_commit + n_k) {
            const long r = u - n_q - n_commit;
            expand_k<HD>(a, (int)(r / a.nkv), (int)(r % a.nkv), lane);
        } else {
            const long r = u - n_q - n_commit - n_k;
            expand_v<HD>(a, (int)(r / a.nkv), (int)(r % a.nkv), base, lane);
        }
    }
}

}  // namespace

int launch_tq_prepare(hipStream_t s, const TqArgs& a0, long max_base) {
    TqArgs a = a0;
    a.inv_sqrt2 = 1.0f / std::sqrt(2.0f);
    if ((a.hd != 64 && a.hd != 128) || a.cap % 16 || a.k.bits < 1 || a.k.bits > 4 || a.v.bits < 1 || a.v.bits > 4) {
        set_error("quantized KV: head_dim must be 64 or 128 and the widths 1..4 bits");
        return TSV_ERR_UNSUPPORTED;
    }
    // a launch that reads its base position on the device (a captured one) is sized for the longest prefix
    const long base = a.base_hint >= 0 ? a.base_hint : max_base;
    const long units = (long)a.m_hint * (a.nq + 2 * a.nkv) + base * a.nkv + ((base + 15) / 16) * a.nkv;
    const int blocks = (int)std::max(1l, std::min((units + 3) / 4, 8192l));
    if (a.hd == 128)
        hipLaunchKernelGGL(k_tq_prepare<128>, dim3(blocks), dim3(256), 0, s, a);
    else
        hipLaunchKernelGGL(k_tq_prepare<64>, dim3(blocks), dim3(256), 0, s, a);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

}  // namespace tsv
