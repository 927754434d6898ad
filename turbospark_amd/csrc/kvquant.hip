// TurboQuant KV rows: the codec's tables (host) and the kernel that runs before the attention of a
// quantized layer.
//
// A quantized layer keeps, per position and kv head, one f32 norm and the packed codebook indices of
// the row's rotated unit vector (crates/compute/src/kv_quant.rs:340-382).  Attention runs in the
// rotated space (crates/compute/src/kv_quant_attention.rs:58-136): q is rotated once with the key
// signs, scores are <q_rot, codebook[idx]> * norm, the values are summed as norm * codebook[idx] and
// the sum is rotated back once with the value signs.  The attention kernel reads the stores directly
// (attn_tq_core.h, which also states their layout); the merge kernel rotates the result back.
//
// The pass's own rows arrive as fp16 in a small staging cache (the staging row of
// crates/runtime/src/kv_write.rs:66-118) and are quantized from there: norm as the f32 sum of squares
// in index order, unit = x * (1 / max(norm, 1e-6)), the butterflies of crates/compute/src/wht.rs:15-29
// in their order with each stage scaled by 1/sqrt(2), one index per coordinate as the count of
// midpoints below it.  Every operation is a single rounded f32 operation in the reference's order, so
// the indices and the norm are the reference's by bits.
#include <algorithm>
#include <cmath>
#include <vector>

#include "attn_tq_core.h"

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

__device__ __forceinline__ long k_at(int cap, int hd, int head, int pos, int d) { return kcache_index(head, pos, d, hd, cap); }
__device__ __forceinline__ long v_at(int cap, int hd, int head, int pos, int d) { return vcache_index(head, pos, d, hd, cap); }

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

// the pass's row at `pos`, kv head `head`: fp16 staging row -> norm and indices in the layer's stores
template <int HD>
__device__ void commit_row(const TqArgs& a, bool value, int pos, int head, int lane, float* s_row, uint32_t* s_words) {
    constexpr int EPL = HD / 64;
    const TqSide& t = value ? a.v : a.k;
    const _Float16* stage = (const _Float16*)(value ? a.vc : a.kc);
    const int slot = pos % a.stage_cap;
    float x[EPL];
#pragma unroll
    for (int j = 0; j < EPL; j++) {
        const int d = lane + 64 * j;
        x[j] = (float)stage[value ? v_at(a.stage_cap, HD, head, slot, d) : k_at(a.stage_cap, HD, head, slot, d)];
        s_row[d] = x[j];
    }
    if (!value && lane < t.words + 1) s_words[lane] = 0;
    lds_order();
    // every lane adds the squares in index order (the reference's sum); the row comes out of LDS sixteen
    // values at a time so that the reads run ahead of the dependent additions
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < HD; i += 16) {
        float4 r[4];
#pragma unroll
        for (int u = 0; u < 4; u++) r[u] = *(const float4*)(s_row + i + 4 * u);
#pragma unroll
        for (int u = 0; u < 4; u++) {
            ss = __fadd_rn(ss, __fmul_rn(r[u].x, r[u].x));
            ss = __fadd_rn(ss, __fmul_rn(r[u].y, r[u].y));
            ss = __fadd_rn(ss, __fmul_rn(r[u].z, r[u].z));
            ss = __fadd_rn(ss, __fmul_rn(r[u].w, r[u].w));
        }
    }
    const float norm = sqrtf(ss);  // correctly rounded, as is the division (the toolchain's default for f32)
    const float inv = 1.0f / fmaxf(norm, 1e-6f);
    float e[EPL];
#pragma unroll
    for (int j = 0; j < EPL; j++) e[j] = __fmul_rn(__fmul_rn(x[j], inv), t.signs[lane + 64 * j]);
    wht<EPL>(e, lane, a.inv_sqrt2);
    const int n_mid = (1 << t.bits) - 1;
    float mid[15];  // the side's midpoints, +inf past the last: the index is the count of midpoints below the coordinate
#pragma unroll
    for (int i = 0; i < 15; i++) {
        const float v = t.mid[i];  // the table holds sixteen slots
        mid[i] = i < n_mid ? v : INFINITY;
    }
    if (lane == 0) (value ? a.store.vn : a.store.kn)[(long)head * a.cap + pos] = norm;
    if (!value) {
        // a K row: packed LSB first (kv_quant.rs:289-312), assembled in LDS
#pragma unroll
        for (int j = 0; j < EPL; j++) {
            uint32_t c = 0;
#pragma unroll
            for (int i = 0; i < 15; i++) c += e[j] > mid[i] ? 1u : 0u;
            const uint32_t bit = (uint32_t)(lane + 64 * j) * (uint32_t)t.bits, w = bit >> 5, off = bit & 31;
            atomicOr(&s_words[w], c << off);
            if (off + t.bits > 32) atomicOr(&s_words[w + 1], c >> (32 - off));
        }
        lds_order();
        if (lane < t.words) a.store.kq[((long)head * a.cap + pos) * t.words + lane] = s_words[lane];
    } else {
        // a V row: index of dimension d into bits (pos % 16) * bits .. of that dimension's group of the block;
        // other rows of the pass own other bits of the same words
        const int gw = tq_v_group_words(t.bits);
        const uint32_t off = (uint32_t)(pos & 15) * (uint32_t)t.bits;
        const uint64_t mask = (uint64_t)n_mid << off;
#pragma unroll
        for (int j = 0; j < EPL; j++) {
            uint32_t c = 0;
#pragma unroll
            for (int i = 0; i < 15; i++) c += e[j] > mid[i] ? 1u : 0u;
            const uint64_t bits = (uint64_t)c << off;
            uint32_t* g = a.store.vq + (((long)head * (a.cap >> 4) + (pos >> 4)) * HD + lane + 64 * j) * gw;
            if ((uint32_t)mask) {
                __hip_atomic_fetch_and(g, ~(uint32_t)mask, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_fetch_or(g, (uint32_t)bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            if (gw == 2 && (uint32_t)(mask >> 32)) {
                __hip_atomic_fetch_and(g + 1, ~(uint32_t)(mask >> 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                __hip_atomic_fetch_or(g + 1, (uint32_t)(bits >> 32), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
        }
    }
    lds_order();
}

// One wave per unit of work: the q rows to rotate, then the pass's K and V rows to quantize.
template <int HD>
__global__ __launch_bounds__(256) void k_tq_prepare(TqArgs a) {
    __shared__ __attribute__((aligned(16))) float s_row[4][HD];
    __shared__ uint32_t s_words[4][HD / 2 + 1];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int m = a.m_hint, base = a.base_hint >= 0 ? a.base_hint : a.vp->base;
    const int n_q = m * a.nq, n_rows = m * a.nkv, total = n_q + 2 * n_rows;
    for (int u = blockIdx.x * 4 + wave; u < total; u += gridDim.x * 4) {
        if (u < n_q) {
            rotate_q<HD>(a, u / a.nq, u % a.nq, lane);
        } else {
            const bool value = u - n_q >= n_rows;
            const int r = u - n_q - (value ? n_rows : 0);
            commit_row<HD>(a, value, base + r / a.nkv, r % a.nkv, lane, s_row[wave], s_words[wave]);
        }
    }
}

}  // namespace

int launch_tq_prepare(hipStream_t s, const TqArgs& a0) {
    TqArgs a = a0;
    a.inv_sqrt2 = 1.0f / std::sqrt(2.0f);
    if ((a.hd != 64 && a.hd != 128) || a.cap % 16 || a.stage_cap % 16 || a.m_hint > a.stage_cap || a.k.bits < 2 || a.k.bits > 4 ||
        a.v.bits < 2 || a.v.bits > 4) {
        set_error("quantized KV: head_dim must be 64 or 128 and the widths 2..4 bits");
        return TSV_ERR_UNSUPPORTED;
    }
    const int units = a.m_hint * (a.nq + 2 * a.nkv);
    const int blocks = std::max(1, (units + 3) / 4);
    if (a.hd == 128)
        hipLaunchKernelGGL(k_tq_prepare<128>, dim3(blocks), dim3(256), 0, s, a);
    else
        hipLaunchKernelGGL(k_tq_prepare<64>, dim3(blocks), dim3(256), 0, s, a);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

namespace {
// Tree compaction over quantized rows (crates/runtime/src/speculative.rs:518-536: the accepted path's rows move to
// consecutive positions): the row at base + path[i] to base + i, in path order.  path is increasing and path[i] >= i,
// so a destination is never a source still to be read.  One thread owns dimension d of a kv head on the V side (its
// groups are its own words, no atomics), word d of the K rows, or one of the two norms.
__global__ void k_tq_gather(const TqKv* __restrict__ stores, int nkv, int hd, int cap, const int32_t* __restrict__ path, int n, int base) {
    const TqKv t = stores[blockIdx.y];
    if (!t.k_bits) return;
    const int id = blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= nkv * hd) return;
    const int head = id / hd, d = id - head * hd;
    const int kw = (hd * t.k_bits + 31) / 32, gw = tq_v_group_words(t.v_bits);
    const uint32_t vmask = (1u << t.v_bits) - 1u;
    for (int i = 0; i < n; i++) {
        const int src = base + path[i], dst = base + i;
        if (src == dst) continue;
        uint32_t* gs = t.vq + (((long)head * (cap >> 4) + (src >> 4)) * hd + d) * gw;
        uint32_t* gd = t.vq + (((long)head * (cap >> 4) + (dst >> 4)) * hd + d) * gw;
        const uint64_t from = gw == 2 ? ((uint64_t)gs[1] << 32) | gs[0] : gs[0];
        uint64_t to = gw == 2 ? ((uint64_t)gd[1] << 32) | gd[0] : gd[0];
        const uint32_t so = (uint32_t)(src & 15) * t.v_bits, dof = (uint32_t)(dst & 15) * t.v_bits;
        to = (to & ~((uint64_t)vmask << dof)) | ((uint64_t)((uint32_t)(from >> so) & vmask) << dof);
        gd[0] = (uint32_t)to;
        if (gw == 2) gd[1] = (uint32_t)(to >> 32);
        if (d < kw) t.kq[((long)head * cap + dst) * kw + d] = t.kq[((long)head * cap + src) * kw + d];
        if (d == kw) t.kn[(long)head * cap + dst] = t.kn[(long)head * cap + src];
        if (d == kw + 1) t.vn[(long)head * cap + dst] = t.vn[(long)head * cap + src];
    }
}
}  // namespace

int launch_tq_gather(hipStream_t s, const TqKv* stores_dev, int n_layers, int nkv, int hd, int cap, const int32_t* path_dev, int n,
                     int base) {
    hipLaunchKernelGGL(k_tq_gather, dim3((nkv * hd + 255) / 256, n_layers), dim3(256), 0, s, stores_dev, nkv, hd, cap, path_dev, n, base);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

size_t tq_kq_bytes(int nkv, int cap, int hd, int k_bits) { return (size_t)nkv * cap * tq_words(hd, k_bits) * 4; }
size_t tq_vq_bytes(int nkv, int cap, int hd, int v_bits) { return (size_t)nkv * (cap / 16) * hd * tq_v_group_words(v_bits) * 4; }

}  // namespace tsv
