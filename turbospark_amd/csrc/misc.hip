// Small per-row kernels of the verify pass: embedding lookup, residual-add + RMSNorm,
// q/k rotation + KV-cache store, KV row gather / read-back.
#include <type_traits>

#include "tsv_internal.h"
#include "x8.h"

namespace tsv {

__device__ __forceinline__ float f16_bits_to_f32(uint16_t h) {
    return (float)__builtin_bit_cast(_Float16, h);
}

// Element e of table row `tok`: the arithmetic of the reference's dequantize_* for the row's storage type.
__device__ __forceinline__ float embed_elem(const uint8_t* __restrict__ raw, int dtype, int hidden, long tok, int e) {
    float v;
    if (dtype == TSV_Q4_K) {
        const uint8_t* blk = raw + (tok * (hidden / 256) + (e >> 8)) * 144;
        const float d = f16_bits_to_f32(*(const uint16_t*)blk);
        const float dmin = f16_bits_to_f32(*(const uint16_t*)(blk + 2));
        const uint8_t* packed = blk + 4;
        const int w = e & 255, g = w >> 6, hi = (w >> 5) & 1, l = w & 31, j = 2 * g + hi;
        int sc, mn;
        if (j < 4) {
            sc = packed[j] & 63;
            mn = packed[j + 4] & 63;
        } else {
            sc = (packed[j + 4] & 0xF) | ((packed[j - 4] >> 6) << 4);
            mn = (packed[j + 4] >> 4) | ((packed[j] >> 6) << 4);
        }
        const uint8_t byte = blk[16 + 32 * g + l];
        const int q = hi ? (byte >> 4) : (byte & 0xF);
        const float dl = d * (float)sc, ml = dmin * (float)mn;
        v = __fsub_rn(__fmul_rn(dl, (float)q), ml);
    } else if (dtype == TSV_Q8_0) {
        const uint8_t* blk = raw + (tok * (hidden / 32) + (e >> 5)) * 34;
        const float d = f16_bits_to_f32(*(const uint16_t*)blk);
        v = (float)(int8_t)blk[2 + (e & 31)] * d;
    } else if (dtype == TSV_Q5_K) {  // q5_k.rs:47-96
        const uint8_t* blk = raw + (tok * (hidden / 256) + (e >> 8)) * 176;
        const float d = f16_bits_to_f32(*(const uint16_t*)blk);
        const float dmin = f16_bits_to_f32(*(const uint16_t*)(blk + 2));
        const uint8_t* packed = blk + 4;
        const int w = e & 255, g = w >> 6, hi = (w >> 5) & 1, l = w & 31, j = 2 * g + hi;
        int sc, mn;
        if (j < 4) {
            sc = packed[j] & 63;
            mn = packed[j + 4] & 63;
        } else {
            sc = (packed[j + 4] & 0xF) | ((packed[j - 4] >> 6) << 4);
            mn = (packed[j + 4] >> 4) | ((packed[j] >> 6) << 4);
        }
        const uint8_t byte = blk[48 + 32 * g + l];
        const int q = (hi ? (byte >> 4) : (byte & 0xF)) + (((blk[16 + l] >> j) & 1) << 4);
        const float dl = d * (float)sc, ml = dmin * (float)mn;
        v = __fsub_rn(__fmul_rn(dl, (float)q), ml);
    } else if (dtype == TSV_Q6_K) {  // q6_k.rs:44-88
        const uint8_t* blk = raw + (tok * (hidden / 256) + (e >> 8)) * 210;
        const int w = e & 255, h = w >> 7, k = (w >> 5) & 3, l = w & 31;
        const int lo = (blk[64 * h + l + 32 * (k & 1)] >> (4 * (k >> 1))) & 0xF;
        const int hi = (blk[128 + 32 * h + l] >> (2 * k)) & 3;
        const float d = f16_bits_to_f32((uint16_t)(blk[208] | (blk[209] << 8)));
        v = d * (float)(int8_t)blk[192 + (w >> 4)] * (float)((lo | (hi << 4)) - 32);
    } else if (dtype == TSV_F16) {
        v = f16_bits_to_f32(((const uint16_t*)raw)[tok * hidden + e]);
    } else if (dtype == TSV_BF16) {
        v = __uint_as_float((uint32_t)((const uint16_t*)raw)[tok * hidden + e] << 16);
    } else {
        v = ((const float*)raw)[tok * hidden + e];
    }
    return v;
}

// ---------------------------------------------------------------- embedding lookup
// One dequantized table row per fed token (crates/runtime/src/real_forward_dispatch.rs:154),
// arithmetic of dequantize_q4_k / dequantize_q8_0.
// The last workgroup of a row (when `cs` is given) fills the row's rotation table instead:
// (cos, sin) of pos * freq, scaled, for every pair index - the same for all layers of the step.
__global__ void k_embed(const uint8_t* __restrict__ raw, int dtype, int hidden, float* __restrict__ x,
                        const VerifyParams* __restrict__ vp, const float* __restrict__ freqs, float mscale,
                        int half, float2* __restrict__ cs, int nblk) {
    const int m = blockIdx.x;
    if (m >= vp->m) return;
    if ((int)blockIdx.y == nblk) {
        const float pos = (float)vp->pos[m];
        for (int i = threadIdx.x; i < half; i += blockDim.x) {
            float sn, c;
            sincosf(pos * freqs[i], &sn, &c);
            cs[m * half + i] = float2{c * mscale, sn * mscale};
        }
        return;
    }
    const long tok = vp->feed[m];
    for (int e = blockIdx.y * blockDim.x + threadIdx.x; e < hidden; e += blockDim.x * nblk)
        x[(long)m * hidden + e] = embed_elem(raw, dtype, hidden, tok, e);
}

int launch_embed(hipStream_t s, const uint8_t* raw, int dtype, int hidden, float* x,
                 const VerifyParams* vp, int m, const float* freqs, float mscale, int half, float2* cs) {
    const int nblk = (hidden + 511) / 512;  // two elements per thread
    hipLaunchKernelGGL(k_embed, dim3(m, nblk + (cs ? 1 : 0)), dim3(256), 0, s, raw, dtype, hidden, x, vp, freqs, mscale,
                       half, cs, nblk);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

// ---------------------------------------------------------------- residual add + RMSNorm
__device__ __forceinline__ float block_sum(float v, float* red) {
    for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o);
    const int wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    if ((threadIdx.x & 63) == 0) red[wave] = v;
    __syncthreads();
    float t = 0.f;
    for (int i = 0; i < nw; i++) t += red[i];
    __syncthreads();
    return t;
}

// x[m] += sum over split-K partials of the previous matmul (fixed order: deterministic), then
// y = x * w / sqrt(mean x^2 + eps) (crates/compute/src/rms_norm.rs:5-14) stored as the next
// matmul's fp16 activation fragments plus the sums of the rounded values over every 32-element
// sub-block (eight neighbouring threads).  One workgroup per row, four consecutive elements per
// thread so every load of a row is issued before the first one is waited on.
__global__ __launch_bounds__(1024) void k_addnorm(float* __restrict__ x, const float* __restrict__ partial,
                                                  int splits, int ldp, const float* __restrict__ w,
                                                  float eps, int hidden, _Float16* __restrict__ xfrag,
                                                  const float* __restrict__ weights,
                                                  const float* __restrict__ bias, X8 x8, int x8_terms, NormBlocks nb) {
    __shared__ float red[16];
    const int m = blockIdx.x;
    // a prompt pass of several 16-row blocks: block blockIdx.y has its own rows, partial sums and fragments
    x += (long)blockIdx.y * nb.x;
    partial += (long)blockIdx.y * nb.partial;
    xfrag = (_Float16*)((char*)xfrag + (long)blockIdx.y * nb.frag);
    float4* xr = (float4*)(x + (long)m * hidden);
    const float4* wr = (const float4*)w;
    const int n4 = hidden >> 2;
    // the norm weights of a thread's first group are asked for now: they come from HBM (nothing
    // else reads them in a step) and would otherwise be waited for after the reduction
    const float4 g_first = (int)threadIdx.x < n4 ? wr[threadIdx.x] : float4{0.f, 0.f, 0.f, 0.f};
    float4 v_first = {0.f, 0.f, 0.f, 0.f};
    float ss = 0.f;
    // The partial sums of a group are loaded with a compile-time count (one of nine straight-line
    // variants, chosen by a uniform branch): all loads are in flight before the first add, where a
    // counted loop would wait for each in turn.
    auto run = [&](auto S) {
        constexpr int NS = decltype(S)::value;
        for (int i = threadIdx.x; i < n4; i += 1024) {
            float4 v = xr[i];
            float4 p[NS > 0 ? NS : 1];
#pragma unroll
            for (int s = 0; s < NS; s++) p[s] = *(const float4*)(partial + ((long)s * 16 + m) * ldp + 4 * i);
            if (weights) {
                // routed experts (families/llama/moe.rs:193-198): the slot outputs are weighted and summed
                // in rank order starting from zero, then added to the stream; product and sum rounded apart
                float4 r = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int s = 0; s < NS; s++) {
                    const float ws = weights[(blockIdx.y * 16 + m) * 8 + s];  // (block b's factors follow block b - 1's)
                    r.x = __fadd_rn(r.x, __fmul_rn(ws, p[s].x));
                    r.y = __fadd_rn(r.y, __fmul_rn(ws, p[s].y));
                    r.z = __fadd_rn(r.z, __fmul_rn(ws, p[s].z));
                    r.w = __fadd_rn(r.w, __fmul_rn(ws, p[s].w));
                }
                v.x = __fadd_rn(v.x, r.x);
                v.y = __fadd_rn(v.y, r.y);
                v.z = __fadd_rn(v.z, r.z);
                v.w = __fadd_rn(v.w, r.w);
            } else {
#pragma unroll
                for (int s = 0; s < NS; s++) {
                    v.x = __fadd_rn(v.x, p[s].x);
                    v.y = __fadd_rn(v.y, p[s].y);
                    v.z = __fadd_rn(v.z, p[s].z);
                    v.w = __fadd_rn(v.w, p[s].w);
                }
                if (bias) {  // the output projection's bias (families/gptoss/mod.rs:16)
                    const float4 b = *(const float4*)(bias + 4 * i);
                    v.x += b.x;
                    v.y += b.y;
                    v.z += b.z;
                    v.w += b.w;
                }
            }
            xr[i] = v;
            if (i == (int)threadIdx.x) v_first = v;
            ss += v.x * v.x + v.y * v.y + v.z * v.z + v.w * v.w;
        }
    };
    switch (splits) {
        case 0: run(std::integral_constant<int, 0>{}); break;
        case 1: run(std::integral_constant<int, 1>{}); break;
        case 2: run(std::integral_constant<int, 2>{}); break;
        case 3: run(std::integral_constant<int, 3>{}); break;
        case 4: run(std::integral_constant<int, 4>{}); break;
        case 5: run(std::integral_constant<int, 5>{}); break;
        case 6: run(std::integral_constant<int, 6>{}); break;
        case 7: run(std::integral_constant<int, 7>{}); break;
        default: run(std::integral_constant<int, 8>{}); break;
    }
    ss = block_sum(ss, red);
    const float inv = 1.0f / sqrtf(ss / (float)hidden + eps);
    float* sums = (float*)((char*)xfrag + xfrag_sum_offset(hidden));
    for (int i = threadIdx.x; i < n4; i += 1024) {
        const bool first = i == (int)threadIdx.x;
        const float4 v = first ? v_first : xr[i], g = first ? g_first : wr[i];
        // elements 4i..4i+3 are one K step of the fragment layout, stored in the order (0, 2, 1, 3)
        typedef _Float16 half4 __attribute__((ext_vector_type(4)));
        typedef uint32_t u32x2_t __attribute__((ext_vector_type(2)));
        half4 h = {(_Float16)(v.x * g.x * inv), (_Float16)(v.z * g.z * inv), (_Float16)(v.y * g.y * inv),
                   (_Float16)(v.w * g.w * inv)};
        // The sums must be those of the stored bits: the matmuls multiply them by the weights' code offsets
        // (up to 1024), so one value rounded differently on the way to the sum than on the way to the store
        // is an error a thousand times its size.  The compiler is free to convert the same product twice, by
        // different instructions; pinning the packed halves in registers leaves it one copy to read.
        u32x2_t hb = __builtin_bit_cast(u32x2_t, h);
        asm volatile("" : "+v"(hb.x), "+v"(hb.y));
        h = __builtin_bit_cast(half4, hb);
        *(half4*)(xfrag + (nb.frag16 ? frag16_index(4 * i, m) : frag_index(4 * i, m))) = h;
        float sum = ((float)h.x + (float)h.y) + ((float)h.z + (float)h.w);
        sum += __shfl_xor(sum, 1);
        sum += __shfl_xor(sum, 2);
        sum += __shfl_xor(sum, 4);
        if ((i & 7) == 0) sums[xsum_index(i >> 3, m)] = sum;
        if (nb.frag2) {  // the same fragments once more, in the other of the two layouts (sums included)
            _Float16* x2 = (_Float16*)((char*)nb.frag2 + (long)blockIdx.y * nb.frag);
            *(half4*)(x2 + (nb.frag16 ? frag_index(4 * i, m) : frag16_index(4 * i, m))) = h;
            if ((i & 7) == 0) ((float*)((char*)x2 + xfrag_sum_offset(hidden)))[xsum_index(i >> 3, m)] = sum;
        }
        if (x8_terms) {
            // the same row as block-scaled fp8 terms, from the unrounded values; the eight threads of a
            // 32-element block are neighbours in one wave (hidden is a multiple of 32)
            float r[4] = {v.x * g.x * inv, v.z * g.z * inv, v.y * g.y * inv, v.w * g.w * inv};
            for (int t = 0; t < x8_terms; t++) {
                float amax = x8_amax4(r);
                amax = fmaxf(amax, __shfl_xor(amax, 1));
                amax = fmaxf(amax, __shfl_xor(amax, 2));
                amax = fmaxf(amax, __shfl_xor(amax, 4));
                const int byte = x8_scale_byte(amax);
                const uint32_t word = x8_term4(r, byte);
                *(uint32_t*)(x8.q + ((size_t)t * 16 + m) * x8.kpad + 4 * i) = word;
                if ((i & 7) == 0) x8.s[((size_t)t * 16 + m) * (x8.kpad >> 5) + (i >> 3)] = (uint8_t)byte;
            }
        }
    }
}

int launch_addnorm(hipStream_t s, float* x, const float* partial, int splits, int ldp, const float* w,
                   float eps, int hidden, uint4* xfrag, int m, const float* weights, const float* bias, const X8* x8,
                   int x8_terms, int blocks, const NormBlocks* nb) {
    if (splits < 0 || splits > 8) {
        set_error("residual add: at most eight partial sums");
        return TSV_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL(k_addnorm, dim3(m, blocks), dim3(1024), 0, s, x, partial, splits, ldp, w, eps, hidden,
                       (_Float16*)xfrag, weights, bias, x8 ? *x8 : X8{}, x8 ? x8_terms : 0, nb ? *nb : NormBlocks{});
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

// ---------------------------------------------------------------- the drafter head's input
// fc's input rows (docs/MTP.md:53-60, families/qwen/mtp.rs:512-590) as matmul fragments, one workgroup per row:
//   [ norm_e(e) ; norm_h(norm_t(h)) ]   e = the embedding row of the row's NEXT token (from the parameter block, or
//   for row 0 from device memory: a proposal the step before picked on the GPU), h = the residual row of the row's
//   position; every norm is x * w / sqrt(mean x^2 + eps) (crates/compute/src/rms_norm.rs:5-14).
// Also the row's rotation table (as the embedding kernel leaves it), and the row of the head's own residual
// stream `x_zero` cleared LAST -- it may be the very row h was read from (a chained step), and fc's partial sums
// are added onto it by the layer's first residual kernel.  Embedding lookup, three norms, the fragment conversion
// and the token hand-over were four launches and a copy before.
__global__ __launch_bounds__(1024) void k_mtp_input(const uint8_t* __restrict__ raw, int dtype, const VerifyParams* __restrict__ vp,
                                                    const int32_t* __restrict__ token_dev, int vocab, const float* h_rows,
                                                    const float* __restrict__ w_e, const float* __restrict__ w_t,
                                                    const float* __restrict__ w_h, float eps, int hidden,
                                                    _Float16* __restrict__ xfrag, float* x_zero,
                                                    const float* __restrict__ freqs, float mscale, int half,
                                                    float2* __restrict__ cs) {
    __shared__ float red[16];
    const int m = blockIdx.x;
    if (m >= vp->m) return;
    long tok = vp->feed[m];
    if (token_dev && m == 0) {
        const int t = *token_dev;
        tok = t < 0 ? 0 : t >= vocab ? vocab - 1 : t;
    }
    const float pos = (float)vp->pos[m];
    for (int i = threadIdx.x; i < half; i += 1024) {
        float sn, c;
        sincosf(pos * freqs[i], &sn, &c);
        cs[m * half + i] = float2{c * mscale, sn * mscale};
    }
    const float* h = h_rows + (long)m * hidden;
    // at most eight elements per thread (hidden <= 8192): kept in registers across the reductions
    float ev[8], hv[8];
    float se = 0.f, sh = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int i = threadIdx.x + 1024 * j;
        ev[j] = i < hidden ? embed_elem(raw, dtype, hidden, tok, i) : 0.f;
        hv[j] = i < hidden ? h[i] : 0.f;
        se += ev[j] * ev[j];
        sh += hv[j] * hv[j];
    }
    se = block_sum(se, red);
    sh = block_sum(sh, red);
    const float inv_e = 1.0f / sqrtf(se / (float)hidden + eps), inv_h = 1.0f / sqrtf(sh / (float)hidden + eps);
    float st = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int i = threadIdx.x + 1024 * j;
        hv[j] = i < hidden ? hv[j] * w_t[i] * inv_h : 0.f;
        st += hv[j] * hv[j];
    }
    st = block_sum(st, red);
    const float inv_t = 1.0f / sqrtf(st / (float)hidden + eps);
    float* sums = (float*)((char*)xfrag + xfrag_sum_offset(2 * hidden));
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const int i = threadIdx.x + 1024 * j;  // hidden is a multiple of 32: whole sub-blocks stay or leave together
        if (i >= hidden) continue;
        const _Float16 he = pinned_half((_Float16)(ev[j] * w_e[i] * inv_e));
        const _Float16 hh = pinned_half((_Float16)(hv[j] * w_h[i] * inv_t));
        xfrag[frag_index(i, m)] = he;
        xfrag[frag_index(hidden + i, m)] = hh;
        float s0 = (float)he, s1 = (float)hh;
        for (int o = 1; o < 32; o <<= 1) {
            s0 += __shfl_xor(s0, o);
            s1 += __shfl_xor(s1, o);
        }
        if ((i & 31) == 0) {
            sums[xsum_index(i >> 5, m)] = s0;
            sums[xsum_index((hidden + i) >> 5, m)] = s1;
        }
        x_zero[(long)m * hidden + i] = 0.f;
    }
}

int launch_mtp_input(hipStream_t s, const uint8_t* raw, int dtype, const VerifyParams* vp, const int32_t* token_dev, int vocab,
                     const float* h_rows, const float* w_e, const float* w_t, const float* w_h, float eps, int hidden, uint4* xfrag,
                     float* x_zero, const float* freqs, float mscale, int half, float2* cs, int m) {
    if (hidden > 8192 || hidden % 32) {
        set_error("drafter head: hidden must be a multiple of 32, at most 8192");
        return TSV_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL(k_mtp_input, dim3(m), dim3(1024), 0, s, raw, dtype, vp, token_dev, vocab, h_rows, w_e, w_t, w_h, eps, hidden,
                       (_Float16*)xfrag, x_zero, freqs, mscale, half, cs);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

__global__ void k_f32_to_xfrag(const float* __restrict__ x, int k, _Float16* __restrict__ xfrag) {
    const int m = blockIdx.y;
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= k) return;  // k is a multiple of 32: whole sub-blocks leave together
    const _Float16 h = pinned_half((_Float16)x[(long)m * k + i]);
    xfrag[frag_index(i, m)] = h;
    float sum = (float)h;
    for (int o = 1; o < 32; o <<= 1) sum += __shfl_xor(sum, o);
    if ((i & 31) == 0) ((float*)((char*)xfrag + xfrag_sum_offset(k)))[xsum_index(i >> 5, m)] = sum;
}

int launch_f32_to_xfrag(hipStream_t s, const float* x, int k, uint4* xfrag, int m) {
    hipLaunchKernelGGL(k_f32_to_xfrag, dim3((k + 255) / 256, m), dim3(256), 0, s, x, k, (_Float16*)xfrag);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

// ---------------------------------------------------------------- rope + KV store
// One wave per (row, head): sums the split-K partials of the fused q/k/v projection, applies
// the optional per-head RMSNorm (families/llama/state.rs:344-347) and the NeoX rotation
// (crates/compute/src/rope.rs:208-256: pairs (i, i + hd/2), angle = position * freq_i), then
// stores q as fp16 rows and K/V straight into the cache slot of that row
// (families/qwen/batched_layers.rs:84-113).  V is stored in 16-position blocks laid out as
// MFMA A-fragments: [hd/16][lane = (pos%16/4)*16 + d%16][pos%4].
__global__ __launch_bounds__(64) void k_rope_kv(RopeKvArgs a) {
    const int m = blockIdx.x, head = blockIdx.y;
    // a prompt pass of several 16-row blocks: block blockIdx.z has its own parameters, partial sums and q rows
    const VerifyParams* vp = a.vp + blockIdx.z;
    a.qkv += (long)blockIdx.z * a.qkv_block_stride;
    a.q16 += (long)blockIdx.z * 16 * a.nq * a.hd;
    // everything the kernel needs from the parameter block is asked for at once
    const int rows = vp->m, rot_pos = vp->pos[m], base = vp->base;
    if (m >= rows) return;
    const int hd = a.hd, half = hd >> 1, i = threadIdx.x;
    const int kind = head < a.nq ? 0 : head < a.nq + a.nkv ? 1 : 2;
    const int h = kind == 0 ? head : kind == 1 ? head - a.nq : head - a.nq - a.nkv;
    const int col = head * hd;  // q heads, then k heads, then v heads: the fused projection's row order
    float x0 = 0.f, x1 = 0.f;
    // where dims i and i + half sit among the head's columns: side by side in the natural order, or -- q and k rows
    // tiled for the rotating epilogue (128-wide heads) -- dims 32 t .. 32 t + 31 in the low half of 64-row tile t and
    // their partners in its high half
    const bool paired = a.paired && kind != 2;
    const int c0 = paired ? (i >> 5) * 64 + (i & 31) : i, c1 = paired ? c0 + 32 : i + half;
    if (i < half) {
        // compile-time split count (a uniform branch picks the variant): every partial is in flight
        // before the first add
        auto sum_splits = [&](auto S) {
            constexpr int NS = decltype(S)::value;
            float p0[NS], p1[NS];
#pragma unroll
            for (int s = 0; s < NS; s++) {
                const float* p = a.qkv + ((long)s * 16 + m) * a.ldq + col;
                p0[s] = p[c0];
                p1[s] = p[c1];
            }
#pragma unroll
            for (int s = 0; s < NS; s++) {
                x0 += p0[s];
                x1 += p1[s];
            }
        };
        switch (a.splits) {
            case 1: sum_splits(std::integral_constant<int, 1>{}); break;
            case 2: sum_splits(std::integral_constant<int, 2>{}); break;
            case 3: sum_splits(std::integral_constant<int, 3>{}); break;
            case 4: sum_splits(std::integral_constant<int, 4>{}); break;
            case 5: sum_splits(std::integral_constant<int, 5>{}); break;
            case 6: sum_splits(std::integral_constant<int, 6>{}); break;
            case 7: sum_splits(std::integral_constant<int, 7>{}); break;
            default: sum_splits(std::integral_constant<int, 8>{}); break;
        }
        if (a.bias) {  // before the rotation (families/gptoss/attn.rs:88-101)
            x0 += a.bias[col + i];
            x1 += a.bias[col + i + half];
        }
    }
    const float* nw = kind == 0 ? a.q_norm : kind == 1 ? a.k_norm : nullptr;
    if (nw) {
        float ss = i < half ? x0 * x0 + x1 * x1 : 0.f;
        for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o);
        const float inv = 1.0f / sqrtf(ss / (float)hd + a.eps);
        if (i < half) {
            x0 = x0 * nw[i] * inv;
            x1 = x1 * nw[i + half] * inv;
        }
    }
    if (i >= half) return;
    if (kind != 2) {
        const float angle = (float)rot_pos * a.freqs[i];
        float sn, cs;
        sincosf(angle, &sn, &cs);
        sn *= a.mscale;
        cs *= a.mscale;
        const float r0 = x0 * cs - x1 * sn;
        const float r1 = x0 * sn + x1 * cs;
        x0 = r0;
        x1 = r1;
    }
    const _Float16 h0 = (_Float16)x0, h1 = (_Float16)x1;
    if (kind == 0) {
        _Float16* q = (_Float16*)a.q16 + ((long)m * a.nq + h) * hd;
        q[i] = h0;
        q[i + half] = h1;
    } else {
        const int pos = (base + m) % a.max_ctx;  // the cache slot of row m (a ring layer wraps at its capacity)
        if (kind == 1) {
            ((_Float16*)a.kc)[kcache_index(h, pos, i, hd, a.max_ctx)] = h0;
            ((_Float16*)a.kc)[kcache_index(h, pos, i + half, hd, a.max_ctx)] = h1;
        } else {
            ((_Float16*)a.vc)[vcache_index(h, pos, i, hd, a.max_ctx)] = h0;
            ((_Float16*)a.vc)[vcache_index(h, pos, i + half, hd, a.max_ctx)] = h1;
        }
    }
}

int launch_rope_kv(hipStream_t s, const RopeKvArgs& a, int m) {
    if (a.splits < 1 || a.splits > 8) {
        set_error("rope: one to eight partial sums");
        return TSV_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL(k_rope_kv, dim3(m, a.nq + 2 * a.nkv, std::max(1, a.blocks)), dim3(64), 0, s, a);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

// ---------------------------------------------------------------- KV row gather / read

// Tree compaction (families/qwen/dflash_tree.rs:106-207): rows of slots path[0..n) move to
// base..base+n.  path is strictly increasing with path[i] >= i, so walking i upward never
// overwrites a row that is still to be read.  One workgroup per (kv head, layer), sequential over i:
// every layer's cache in one launch.
__global__ void k_kv_gather(uint16_t* const* caches, const int32_t* caps, int hd, const int32_t* path, int n, int base) {
    // grid (kv heads, layers): caches[2 * layer] is the layer's K buffer, [2 * layer + 1] its V buffer,
    // caps[layer] the positions it holds (a ring layer wraps there)
    uint16_t* kc = caches[2 * blockIdx.y];
    uint16_t* vc = caches[2 * blockIdx.y + 1];
    const int max_ctx = caps[blockIdx.y];
    if (max_ctx == 0) return;  // a layer without fp16 rows (quantized KV)
    const int h = blockIdx.x, d = threadIdx.x;
    for (int i = 0; i < n; i++) {
        const int src = (base + path[i]) % max_ctx, dst = (base + i) % max_ctx;
        if (src == dst) continue;
        if (d < hd) {
            kc[kcache_index(h, dst, d, hd, max_ctx)] = kc[kcache_index(h, src, d, hd, max_ctx)];
            vc[vcache_index(h, dst, d, hd, max_ctx)] = vc[vcache_index(h, src, d, hd, max_ctx)];
        }
    }
}

int launch_kv_gather(hipStream_t s, uint16_t* const* caches_dev, const int32_t* caps_dev, int n_layers, int nkv, int hd,
                     const int32_t* path_dev, int n, int base) {
    hipLaunchKernelGGL(k_kv_gather, dim3(nkv, n_layers), dim3(128), 0, s, caches_dev, caps_dev, hd, path_dev, n, base);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

__global__ void k_kv_read(const uint16_t* kc, const uint16_t* vc, int nkv, int hd, int max_ctx, int pos0,
                          uint16_t* k_out, uint16_t* v_out) {
    const int p = blockIdx.x, h = blockIdx.y, d = threadIdx.x;
    if (d >= hd) return;
    const long o = ((long)p * nkv + h) * hd + d;
    const int pos = (pos0 + p) % max_ctx;
    k_out[o] = kc[kcache_index(h, pos, d, hd, max_ctx)];
    v_out[o] = vc[vcache_index(h, pos, d, hd, max_ctx)];
}

__global__ void k_kv_fill(uint16_t* kc, uint16_t* vc, int nkv, int hd, int max_ctx, int pos0,
                          const uint16_t* k_in, const uint16_t* v_in) {
    const int p = blockIdx.x, h = blockIdx.y, d = threadIdx.x;
    if (d >= hd) return;
    const long o = ((long)p * nkv + h) * hd + d;
    const int pos = (pos0 + p) % max_ctx;
    kc[kcache_index(h, pos, d, hd, max_ctx)] = k_in[o];
    vc[vcache_index(h, pos, d, hd, max_ctx)] = v_in[o];
}

int launch_kv_fill(hipStream_t s, uint16_t* kc, uint16_t* vc, int nkv, int hd, int max_ctx, int pos0, int n,
                   const uint16_t* k_in, const uint16_t* v_in) {
    hipLaunchKernelGGL(k_kv_fill, dim3(n, nkv), dim3(128), 0, s, kc, vc, nkv, hd, max_ctx, pos0, k_in, v_in);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

int launch_kv_read(hipStream_t s, const uint16_t* kc, const uint16_t* vc, int nkv, int hd, int max_ctx,
                   int pos0, int n, uint16_t* k_out, uint16_t* v_out) {
    hipLaunchKernelGGL(k_kv_read, dim3(n, nkv), dim3(128), 0, s, kc, vc, nkv, hd, max_ctx, pos0, k_out, v_out);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

}  // namespace tsv
