// Flash-decoding split-KV GQA attention for a verify pass on gfx950.
//
// Replaces the reference's per-row loop of split-KV decode dispatches
// (crates/runtime/src/families/qwen/batched_layers.rs:409-430 over
// crates/gpu/src/attention_decode.rs:1092-1363, tree variant :1153-1230); arithmetic contract
// crates/compute/src/attention.rs:53-137.  Differences by design:
//  * ALL rows of the pass (and all q heads of a GQA group) share ONE read of K and V: the
//    (row, q-head-in-group) pairs are the 16-wide N operand of the MFMA, so the KV bytes are
//    read once per layer instead of once per row;
//  * the causal / tree mask over the drafted suffix is a 16-bit ancestor set per row;
//  * S^T = K Q^T is computed with v_mfma_f32_16x16x32_f16 (K positions as the M operand), whose
//    accumulator layout (lane: row j, positions 4*kg..4*kg+3) is exactly the B-operand layout
//    of v_mfma_f32_16x16x16_f16, so O^T += V^T P^T needs no data movement; V is stored in the
//    cache pre-arranged as that MFMA's A fragments.
#include <algorithm>

#include "attn_tq_core.h"

namespace tsv {

int attn_chunks(int nkv) {
    int n = 256 / nkv;
    if (n < 1) n = 1;
    if (n > 64) n = 64;
    return n;
}

// blocks in flight per wave when a workgroup holds two row tiles: two at 128-wide heads (a third block's
// registers would spill), three at 64-wide ones
#ifndef TSV_ATTN_STAGES2_HD128
#define TSV_ATTN_STAGES2_HD128 2
#endif
#ifndef TSV_ATTN_STAGES2_HD64
#define TSV_ATTN_STAGES2_HD64 3
#endif

// Eight waves per workgroup share a chunk of the context (attn_core.h).
template <int HD, int RT, int STAGES>
__global__ __launch_bounds__(512) void k_attn_partial(AttnArgs a, int G, int R) {
    extern __shared__ float xch[];  // [4 slots][PER_LANE values][64 lanes]
    if (a.xcd_groups) {  // several row groups of a verify pass: placed by die
        int chunk, kvh, grp;
        if (attn_grid_place(a, blockIdx.x, chunk, kvh, grp)) attn_partial_body<HD, RT, STAGES, false>(a, G, R, chunk, kvh, grp * RT, xch);
        return;
    }
    // grid z: row groups of the pass, times the 16-row blocks of a prompt pass
    const int groups = gridDim.z / max(a.blocks, 1), blk = blockIdx.z / groups, grp = blockIdx.z - blk * groups;
    if (a.blocks > 1) {
        const AttnArgs v = attn_block_view(a, blk);
        attn_partial_body<HD, RT, STAGES, false>(v, G, R, blockIdx.x, blockIdx.y, grp * RT, xch);
        return;
    }
    attn_partial_body<HD, RT, STAGES, false>(a, G, R, blockIdx.x, blockIdx.y, grp * RT, xch);
}

// A pass of more than two row tiles: TG tile groups side by side in one workgroup (attn_core.h), one read of the
// chunk's K / V blocks out of the L2 for all of them.  Grid (chunks, kv heads, 16-row blocks of a prompt pass).
template <int HD, int RT, int STAGES, int TG>
__global__ __launch_bounds__(64 * TG * attn_phases(TG)) void k_attn_partial_groups(AttnArgs a, int G, int R) {
    extern __shared__ float xch[];
    if (a.blocks > 1) {
        const AttnArgs v = attn_block_view(a, blockIdx.z);
        attn_partial_body<HD, RT, STAGES, false, TG>(v, G, R, blockIdx.x, blockIdx.y, 0, xch);
        return;
    }
    attn_partial_body<HD, RT, STAGES, false, TG>(a, G, R, blockIdx.x, blockIdx.y, 0, xch);
}

// The same pass over a layer that keeps quantized rows (attn_tq_core.h)
template <int HD, int RT, int KB, int VB>
__global__ __launch_bounds__(512) void k_attn_partial_tq(AttnArgs a, int G, int R) {
    extern __shared__ float xch[];
    __shared__ uint32_t s_kpair[1 << (2 * KB)], s_vpair[1 << (2 * VB)];
    tq_fill_pairs(s_kpair, a.tq.k_cb, KB, threadIdx.x, 512);
    tq_fill_pairs(s_vpair, a.tq.v_cb, VB, threadIdx.x, 512);
    __syncthreads();
    // blocks in flight: three, two where the three-bit fields' extra words would push the registers past 256
    constexpr int STAGES = (HD == 128 && RT == 2 && KB == 3 && VB == 3) ? 2 : 3;
    if (a.xcd_groups) {
        int chunk, kvh, grp;
        if (attn_grid_place(a, blockIdx.x, chunk, kvh, grp))
            attn_partial_body_tq<HD, RT, STAGES, KB, VB>(a, G, R, chunk, kvh, grp * RT, xch, s_kpair, s_vpair);
        return;
    }
    // grid z: row groups of the pass, times the 16-row blocks of a prompt pass
    const int groups = gridDim.z / max(a.blocks, 1), blk = blockIdx.z / groups, grp = blockIdx.z - blk * groups;
    if (a.blocks > 1) {
        const AttnArgs v = attn_block_view(a, blk);
        attn_partial_body_tq<HD, RT, STAGES, KB, VB>(v, G, R, blockIdx.x, blockIdx.y, grp * RT, xch, s_kpair, s_vpair);
        return;
    }
    attn_partial_body_tq<HD, RT, STAGES, KB, VB>(a, G, R, blockIdx.x, blockIdx.y, grp * RT, xch, s_kpair, s_vpair);
}

// Merge the chunk partials (crates/gpu/src/shaders/attention.metal:122-140 semantics:
// m* = max m_c, D = sum l_c e^{m_c-m*}, O = sum O_c e^{m_c-m*}, out = O / D) and store the row
// as fp16 activation fragments (and sub-block sums) of the output projection (K index =
// q_head*hd + d).  The first
// wave turns the (m_c, l_c) pairs into per-chunk weights once; every thread then sums its
// output element over the chunks with independent loads.
// NCH > 0: the chunk count as a compile-time constant -- every thread then asks for its output
// element of all chunks before the (m, l) pairs are looked at (the two groups of loads do not
// depend on each other), and the kernel is one memory latency instead of two.  NCH == 0: any count.
template <int NCH, bool UNROT>
__global__ void k_attn_combine(AttnArgs a0, int G, int R) {
    const AttnArgs a = a0.blocks > 1 ? attn_block_view(a0, blockIdx.z) : a0;
    __shared__ float wgt[64];
    __shared__ float s_den;
    const int m = blockIdx.x, qh = blockIdx.y, d = threadIdx.x;
    const int hd = a.hd, nch = NCH > 0 ? NCH : a.nch;
    const int h = qh / G, g = qh - h * G, r = m * G + g;
    const float* po = a.part_o + ((long)h * nch * R + r) * hd + min(d, hd - 1);
    const long stride = (long)R * hd;
    float pre[NCH > 0 ? NCH : 1];
    if (NCH > 0) {
#pragma unroll
        for (int c = 0; c < NCH; c++) pre[c] = po[c * stride];
    }
    if (d < 64) {
        float mc = -INFINITY, lc = 0.f;
        if (d < nch) {
            const long slot = ((long)h * nch + d) * R + r;
            mc = a.part_ml[slot * 2];
            lc = a.part_ml[slot * 2 + 1];
        }
        float mx = mc;
        for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
        // the sink joins the maximum and the denominator, never the numerator
        // (crates/compute/src/attention.rs:94-105)
        const float sink = a.sinks ? a.sinks[qh] : -INFINITY;
        mx = fmaxf(mx, sink);
        const float w = mc > -INFINITY ? __expf(mc - mx) : 0.f;
        float den = lc * w;
        for (int o = 32; o > 0; o >>= 1) den += __shfl_xor(den, o);
        if (a.sinks) den += __expf(sink - mx);
        wgt[d] = w;
        if (d == 0) s_den = den;
    }
    __syncthreads();
    if (d >= hd) return;
    float num = 0.f;
    if (NCH > 0) {
#pragma unroll
        for (int c = 0; c < NCH; c++) num = fmaf(wgt[c], pre[c], num);
    } else {
#pragma unroll 8
        for (int c = 0; c < nch; c++) num = fmaf(wgt[c], po[c * stride], num);
    }
    float res = num / s_den;
    if (UNROT) {
        // the sum was taken over rotated value rows: back through the normalized Hadamard transform
        // (crates/compute/src/wht.rs:15-29, stage h pairs d with d + h) and the value signs
        __shared__ float s_h[128];
        const float c = 0.70710678118654752440f;
        for (int st = 1; st < hd; st <<= 1) {
            s_h[d] = res;
            __syncthreads();
            const float other = s_h[d ^ st];
            __syncthreads();
            res = ((d & st) ? other - res : res + other) * c;
        }
        res *= a.unrot[d];
    }
    const _Float16 o16 = (_Float16)res;
    const int kk = qh * hd + d;
    ((_Float16*)a.xfrag)[a.frag16 ? frag16_index(kk, m) : frag_index(kk, m)] = o16;
    // sum of each 32-element sub-block of the output projection's input (32 neighbouring threads)
    float sum = (float)o16;
    for (int o = 1; o < 32; o <<= 1) sum += __shfl_xor(sum, o);
    if ((d & 31) == 0) ((float*)((char*)a.xfrag + xfrag_sum_offset(a.nq * hd)))[xsum_index(kk >> 5, m)] = sum;
}

template <int HD, int RT, int STAGES>
static int launch_partial(hipStream_t s, const AttnArgs& a, int G, int R, int groups) {
    constexpr int PER_LANE = RT * (HD / 16) * 4 + 2 * RT;
    const size_t lds = (size_t)4 * 64 * PER_LANE * 4;
    static bool raised = false;  // more than 64 KiB of dynamic LDS has to be allowed once per kernel
    if (lds > 65536 && !raised) {
        TSV_HIP(hipFuncSetAttribute((const void*)k_attn_partial<HD, RT, STAGES>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)lds));
        raised = true;
    }
    const dim3 grid = a.xcd_groups ? dim3(attn_grid_size(a.nch * a.nkv, groups)) : dim3(a.nch, a.nkv, groups * std::max(a.blocks, 1));
    hipLaunchKernelGGL((k_attn_partial<HD, RT, STAGES>), grid, dim3(512), lds, s, a, G, R);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

template <int HD, int RT, int STAGES, int TG>
static int launch_partial_groups(hipStream_t s, const AttnArgs& a, int G, int R) {
    constexpr int PER_LANE = RT * (HD / 16) * 4 + 2 * RT, NW = attn_phases(TG), SLOTS = NW < 4 ? NW : 4;
    const size_t lds = (size_t)TG * SLOTS * 64 * PER_LANE * 4;
    static bool raised = false;  // more than 64 KiB of dynamic LDS has to be allowed once per kernel
    if (lds > 65536 && !raised) {
        TSV_HIP(hipFuncSetAttribute((const void*)k_attn_partial_groups<HD, RT, STAGES, TG>,
                                    hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        raised = true;
    }
    hipLaunchKernelGGL((k_attn_partial_groups<HD, RT, STAGES, TG>), dim3(a.nch, a.nkv, std::max(a.blocks, 1)), dim3(64 * TG * NW),
                       lds, s, a, G, R);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

template <int HD>
static int launch_combine(hipStream_t s, const AttnArgs& a, int m, int G, int R);

template <int HD, int RT, int KB, int VB>
static int launch_partial_tq(hipStream_t s, const AttnArgs& a, int G, int R, int groups) {
    constexpr int PER_LANE = RT * (HD / 16) * 4 + 2 * RT;
    const size_t lds = (size_t)4 * 64 * PER_LANE * 4;
    static bool raised = false;
    if (lds > 60000 && !raised) {  // with the pair tables beside it the exchange area passes 64 KiB
        TSV_HIP(hipFuncSetAttribute((const void*)k_attn_partial_tq<HD, RT, KB, VB>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)lds));
        raised = true;
    }
    const dim3 grid = a.xcd_groups ? dim3(attn_grid_size(a.nch * a.nkv, groups)) : dim3(a.nch, a.nkv, groups * std::max(a.blocks, 1));
    hipLaunchKernelGGL((k_attn_partial_tq<HD, RT, KB, VB>), grid, dim3(512), lds, s, a, G, R);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}
template <int HD, int RT>
static int launch_partial_tq_widths(hipStream_t s, const AttnArgs& a, int G, int R, int groups) {
    const int kb = a.tq.k_bits, vb = a.tq.v_bits;
    if (kb == 4 && vb == 4) return launch_partial_tq<HD, RT, 4, 4>(s, a, G, R, groups);
    if (kb == 3 && vb == 4) return launch_partial_tq<HD, RT, 3, 4>(s, a, G, R, groups);
    if (kb == 3 && vb == 3) return launch_partial_tq<HD, RT, 3, 3>(s, a, G, R, groups);
    if (kb == 2 && vb == 2) return launch_partial_tq<HD, RT, 2, 2>(s, a, G, R, groups);
    set_error("attention: no kernel for these KV quantization widths");
    return TSV_ERR_UNSUPPORTED;
}

template <int HD>
static int launch_hd(hipStream_t s, const AttnArgs& a0, int m, int G, int R) {
    const int trt = (R + 15) / 16;
    // more than 32 (row, q head) pairs: groups of 32, each re-reading K and V (from L2)
    const int groups = trt <= 2 ? 1 : (trt + 1) / 2;
    // about one workgroup per compute unit: the chunk count shrinks as the row groups multiply
    // (fewer, longer chunks also mean fewer partial results for the merge to read)
    AttnArgs a = a0;
    a.nch = std::max(std::min(a0.nch, 8), std::min(a0.nch, 256 / (a0.nkv * groups * std::max(a0.blocks, 1))));
    // Several row groups of a verify pass read the same K / V: they are placed on one die.  A workgroup fills a
    // compute unit (eight waves at two per SIMD) and a die has 32 of them: no die may be handed more than 32
    // workgroups, or its last one waits for a whole workgroup to end (26 against 18 us at 21 chunks x 4 heads x 3)
    a.xcd_groups = (groups > 1 && a0.blocks <= 1) ? groups : 0;
    if (a.xcd_groups) a.nch = std::max(std::min(a0.nch, 8), std::min(a0.nch, 8 * (32 / groups) / a0.nkv));
    int rc;
    if (a.tq.k_bits) {
        if (a.window || a.ring || !a.unrot) {
            set_error("attention: quantized rows go with full attention and a linear cache");
            return TSV_ERR_UNSUPPORTED;
        }
        rc = trt <= 1 ? launch_partial_tq_widths<HD, 1>(s, a, G, R, 1) : launch_partial_tq_widths<HD, 2>(s, a, G, R, groups);
    } else if (trt <= 1)
        rc = launch_partial<HD, 1, 3>(s, a, G, R, 1);
    else if (trt <= 2)
        rc = launch_partial<HD, 2, (HD == 128 ? TSV_ATTN_STAGES2_HD128 : TSV_ATTN_STAGES2_HD64)>(s, a, G, R, 1);
    else {
        // more row tiles than a wave holds: tile groups inside one workgroup, about one workgroup per compute unit
        a.xcd_groups = 0;
        a.nch = std::max(1, std::min(a0.nch, 256 / (a0.nkv * std::max(a0.blocks, 1))));
        // (64 chunks at four KV heads would fill the chip, but what the partial pass wins the merge loses reading
        // twice the partial results: 10.9 + 6.0 us against 12.9 + 4.1 us at the Qwen3-30B-A3B shape)
        if (a.nch > 32) a.nch = 32;
        constexpr int ST = HD == 128 ? TSV_ATTN_STAGES2_HD128 : TSV_ATTN_STAGES2_HD64;
        if (HD == 64 && trt >= 7)
            rc = launch_partial_groups<HD, (HD == 64 ? 4 : 2), 2, 2>(s, a, G, R);
        else if (HD == 64 && trt >= 5)
            rc = launch_partial_groups<HD, (HD == 64 ? 3 : 2), 2, 2>(s, a, G, R);
        else if (trt <= 4)
            rc = launch_partial_groups<HD, 2, ST, 2>(s, a, G, R);
        else if (trt <= 6)
            rc = launch_partial_groups<HD, 2, ST, 3>(s, a, G, R);
        else
            rc = launch_partial_groups<HD, 2, ST, 4>(s, a, G, R);
    }
    if (rc) return rc;
    return launch_combine<HD>(s, a, m, G, R);
}

template <int HD>
static int launch_combine(hipStream_t s, const AttnArgs& a, int m, int G, int R) {
    const dim3 cgrid(m, a.nq, std::max(a.blocks, 1)), cblock(HD < 64 ? 64 : HD);
    // the chunk count as a compile-time constant puts every partial's load in flight before the
    // first add (a counted loop waits on each in turn); the sum runs in the same order either way
    // UNROT: the variant that rotates each head's result back (quantized KV rows); the other one is unchanged code
#define TSV_COMBINE(N)                                                                         \
    case N:                                                                                    \
        if (a.unrot)                                                                           \
            hipLaunchKernelGGL((k_attn_combine<N, true>), cgrid, cblock, 0, s, a, G, R);       \
        else                                                                                   \
            hipLaunchKernelGGL((k_attn_combine<N, false>), cgrid, cblock, 0, s, a, G, R);      \
        break;
    switch (a.nch) {
        TSV_COMBINE(1) TSV_COMBINE(2) TSV_COMBINE(3) TSV_COMBINE(4) TSV_COMBINE(5) TSV_COMBINE(6) TSV_COMBINE(7) TSV_COMBINE(8)
        TSV_COMBINE(9) TSV_COMBINE(10) TSV_COMBINE(11) TSV_COMBINE(12) TSV_COMBINE(13) TSV_COMBINE(14) TSV_COMBINE(15)
        TSV_COMBINE(16) TSV_COMBINE(17) TSV_COMBINE(18) TSV_COMBINE(19) TSV_COMBINE(20) TSV_COMBINE(21) TSV_COMBINE(22)
        TSV_COMBINE(23) TSV_COMBINE(24) TSV_COMBINE(25) TSV_COMBINE(26) TSV_COMBINE(27) TSV_COMBINE(28) TSV_COMBINE(29)
        TSV_COMBINE(30) TSV_COMBINE(31) TSV_COMBINE(32)
        default:
            if (a.unrot)
                hipLaunchKernelGGL((k_attn_combine<0, true>), cgrid, cblock, 0, s, a, G, R);
            else
                hipLaunchKernelGGL((k_attn_combine<0, false>), cgrid, cblock, 0, s, a, G, R);
            break;
    }
#undef TSV_COMBINE
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

// the merge alone, over partials some other kernel left (a.nch chunks)
int launch_attention_merge(hipStream_t s, const AttnArgs& a, int m) {
    const int G = a.nq / a.nkv, R = m * G;
    return a.hd == 128 ? launch_combine<128>(s, a, m, G, R) : launch_combine<64>(s, a, m, G, R);
}

int launch_attention(hipStream_t s, const AttnArgs& a, int m) {
    const int G = a.nq / a.nkv, R = m * G;
    if (a.hd == 128) return launch_hd<128>(s, a, m, G, R);
    if (a.hd == 64) return launch_hd<64>(s, a, m, G, R);
    set_error("attention: head_dim must be 64 or 128");
    return TSV_ERR_UNSUPPORTED;
}

}  // namespace tsv
