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

#include "tsv_internal.h"

namespace tsv {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

int attn_chunks(int nkv) {
    int n = 256 / nkv;
    if (n < 1) n = 1;
    if (n > 64) n = 64;
    return n;
}

// The library is compiled with -ffp-contract=off and every fused multiply-add here is written out:
// left to itself the compiler contracts a * b + c * d one way in one template instantiation and the
// other way in the next, and a row's bits would then depend on how many rows share its pass.
//
// One (m, l, O) running state merged into another (flash-decoding rescale).
template <int RT, int VT>
__device__ __forceinline__ void merge_state(float (&mrun)[RT], float (&lrun)[RT], float4v (&O)[RT][VT], const float* src) {
    // `src` points at this lane's column of a [values][64 lanes] slot: consecutive lanes touch
    // consecutive LDS banks
#pragma unroll
    for (int t = 0; t < RT; t++) {
        const float m1 = src[64 * (2 * t)], l1 = src[64 * (2 * t + 1)];
        const float mnew = fmaxf(mrun[t], m1);
        if (mnew > -INFINITY) {
            const float a0 = __expf(mrun[t] - mnew), a1 = __expf(m1 - mnew);
            lrun[t] = fmaf(lrun[t], a0, l1 * a1);
#pragma unroll
            for (int d = 0; d < VT; d++)
#pragma unroll
                for (int i = 0; i < 4; i++) O[t][d][i] = fmaf(O[t][d][i], a0, src[64 * (2 * RT + (t * VT + d) * 4 + i)] * a1);
            mrun[t] = mnew;
        }
    }
}
template <int RT, int VT>
__device__ __forceinline__ void store_state(const float (&mrun)[RT], const float (&lrun)[RT], const float4v (&O)[RT][VT],
                                            float* dst) {
#pragma unroll
    for (int t = 0; t < RT; t++) {
        dst[64 * (2 * t)] = mrun[t];
        dst[64 * (2 * t + 1)] = lrun[t];
#pragma unroll
        for (int d = 0; d < VT; d++)
#pragma unroll
            for (int i = 0; i < 4; i++) dst[64 * (2 * RT + (t * VT + d) * 4 + i)] = O[t][d][i];
    }
}

// Eight waves per workgroup share a chunk of the context, each walking every eighth 16-position
// block with up to STAGES blocks of K and V in flight.
template <int HD, int RT, int STAGES>
__global__ __launch_bounds__(512) void k_attn_partial(AttnArgs a, int G, int R) {
    constexpr int NW = 8;
    constexpr int KS = HD / 32;  // K steps of the score MFMA
    constexpr int VT = HD / 16;  // output tiles along head_dim
    constexpr int PER_LANE = RT * VT * 4 + 2 * RT;
    extern __shared__ float xch[];  // [4 slots][PER_LANE values][64 lanes]

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 15, kg = lane >> 4;
    const int chunk = blockIdx.x, h = blockIdx.y, rt0 = blockIdx.z * RT;
    const VerifyParams* vp = a.vp;
    const int M = a.base_hint >= 0 ? a.m_hint : vp->m, base = a.base_hint >= 0 ? a.base_hint : vp->base, kvlen = base + M;
    const int nblk = (kvlen + 15) >> 4;
    // sliding window (families/gptoss/attn.rs:120-137): a row at sequence length n sees positions
    // n - window .. n - 1.  The window exceeds the pass width, so every row keeps its whole drafted
    // suffix and the cut falls in the committed prefix: blocks before the first row's cut are not
    // read at all, the few blocks where the rows' cuts differ are masked per row.
    const int window = a.window;
    const int bfirst = window > 0 ? max(base + 1 - window, 0) >> 4 : 0;
    const int bpc = (nblk - bfirst + a.nch - 1) / a.nch;
    const int b0 = bfirst + chunk * bpc, b1 = min(b0 + bpc, nblk);
    const int cut_end = window > 0 ? base + M - window : 0;  // positions from here on are inside every row's window
    const float scale = a.scale;
    const uint32_t mmask = (1u << M) - 1u;  // slots that exist in this pass

    // query fragments and per-row ancestor sets
    uint4 qf[RT][KS];
    uint32_t anc[RT];
    int lo[RT];  // first visible position of the row (window)
#pragma unroll
    for (int t = 0; t < RT; t++) {
        const int r = (rt0 + t) * 16 + j;
        anc[t] = 0xFFFFu;
        lo[t] = 0;
        if (r < R) {
            const int mrow = r / G, g = r - mrow * G;
            anc[t] = vp->anc[mrow];
            if (window > 0) lo[t] = vp->pos[mrow] + 1 - window;
            const _Float16* q = (const _Float16*)a.q16 + ((long)mrow * a.nq + h * G + g) * HD + 8 * kg;
#pragma unroll
            for (int s = 0; s < KS; s++) qf[t][s] = *(const uint4*)(q + 32 * s);
        } else {
#pragma unroll
            for (int s = 0; s < KS; s++) qf[t][s] = make_uint4(0, 0, 0, 0);
        }
    }

    float mrun[RT], lrun[RT];
    float4v O[RT][VT];
#pragma unroll
    for (int t = 0; t < RT; t++) {
        mrun[t] = -INFINITY;
        lrun[t] = 0.f;
#pragma unroll
        for (int d = 0; d < VT; d++) O[t][d] = float4v{0.f, 0.f, 0.f, 0.f};
    }

    // this head's K rows and V blocks as buffers that end after block b1 - 1
    const uint32_t blk_bytes = 16 * HD * 2;
    const __amdgpu_buffer_rsrc_t krs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)((const _Float16*)a.kc + (long)h * a.max_ctx * HD), 0, (int)(b1 * blk_bytes), 0x00027000);
    const __amdgpu_buffer_rsrc_t vrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)((const _Float16*)a.vc + (long)h * (a.max_ctx >> 4) * (HD * 16)), 0, (int)(b1 * blk_bytes), 0x00027000);
    struct Blk {
        u32x4 kf[KS];
        u32x2 vf[VT];
    };
    const uint32_t koff = (uint32_t)(j * HD + 8 * kg) * 2, voff = (uint32_t)lane * 8;
    const int nb = b1 > b0 + wave ? (b1 - b0 - wave + NW - 1) / NW : 0;  // blocks of this wave
    auto fetch = [&](Blk& st, int i) {  // block i of this wave's run
        const uint32_t bo = (uint32_t)(b0 + wave + NW * i) * blk_bytes;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < KS; s++) st.kf[s] = __builtin_amdgcn_raw_buffer_load_b128(krs, bo + koff + 64 * s, 0, 0);
#pragma unroll
        for (int d = 0; d < VT; d++) st.vf[d] = __builtin_amdgcn_raw_buffer_load_b64(vrs, bo + voff + 512 * d, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    auto consume = [&](const Blk& st, int i) {
        const int p0 = (b0 + wave + NW * i) << 4;
        const bool tail = p0 + 16 > base;
#pragma unroll
        for (int t = 0; t < RT; t++) {
            float4v S = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < KS; s++)
                S = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, st.kf[s]),
                                                           __builtin_bit_cast(half8, qf[t][s]), S, 0, 0, 0);
            // Visibility of this lane's four positions as a 4-bit word, computed without
            // branches: bit (slot + 16) of `w` says whether cache slot base+slot is visible
            // (the 16 low bits stand for prefix positions, always visible).
            uint32_t vis4 = 0xFu;
            if (tail) {
                const uint64_t w = ((uint64_t)(anc[t] & mmask) << 16) | 0xFFFFull;
                vis4 = (uint32_t)(w >> (p0 + 4 * kg - base + 16)) & 0xFu;  // shift in [1, 47]
            }
            if (p0 < cut_end) {  // some row's window starts inside or after this block
                const int d = lo[t] - (p0 + 4 * kg);  // this lane's positions below index d are outside
                vis4 &= d <= 0 ? 0xFu : d >= 4 ? 0u : (0xFu << d) & 0xFu;
            }
            float sc[4];
#pragma unroll
            for (int i4 = 0; i4 < 4; i4++) sc[i4] = ((vis4 >> i4) & 1u) ? S[i4] * scale : -INFINITY;
            float mb = fmaxf(fmaxf(sc[0], sc[1]), fmaxf(sc[2], sc[3]));
            mb = fmaxf(mb, __shfl_xor(mb, 16));
            mb = fmaxf(mb, __shfl_xor(mb, 32));
            const float mnew = fmaxf(mrun[t], mb);
            float alpha = 1.f;
            half4 P = {0, 0, 0, 0};
            if (mnew > -INFINITY) {
                alpha = __expf(mrun[t] - mnew);
                float ps = 0.f;
#pragma unroll
                for (int i4 = 0; i4 < 4; i4++) {
                    const float p = __expf(sc[i4] - mnew);
                    ps += p;
                    P[i4] = (_Float16)p;
                }
                lrun[t] = fmaf(lrun[t], alpha, ps);
                mrun[t] = mnew;
            }
#pragma unroll
            for (int d = 0; d < VT; d++) {
                O[t][d] *= alpha;
                O[t][d] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4, st.vf[d]), P, O[t][d], 0, 0, 0);
            }
        }
    };
    // Short runs are straight-line code (every load issued before the first wait, no load the run
    // does not need); longer ones keep STAGES blocks in flight, with unconditional loads in the
    // steady state so the compiler waits on the oldest block only.
    if (nb == 1) {
        Blk st;
        fetch(st, 0);
        consume(st, 0);
    } else if (nb == 2) {
        Blk s0, s1;
        fetch(s0, 0);
        fetch(s1, 1);
        consume(s0, 0);
        consume(s1, 1);
    } else if (nb >= STAGES) {
        Blk st[STAGES];
#pragma unroll
        for (int s = 0; s < STAGES; s++) fetch(st[s], s);
        int i = 0;
        for (; i + 2 * STAGES <= nb; i += STAGES) {
#pragma unroll
            for (int s = 0; s < STAGES; s++) {
                consume(st[s], i + s);
                fetch(st[s], i + s + STAGES);
            }
        }
#pragma unroll
        for (int s = 0; s < STAGES; s++) {
            if (i + s < nb) {
                consume(st[s], i + s);
                if (i + s + STAGES < nb) fetch(st[s], i + s + STAGES);
            }
        }
        i += STAGES;
#pragma unroll
        for (int s = 0; s < STAGES; s++)
            if (i + s < nb) consume(st[s], i + s);
    }

    // fold the eight waves' running (m, l, O): 4..7 into 0..3, then 1..3 into 0
    float* mine = xch + (wave & 3) * 64 * PER_LANE + lane;
    if (wave >= 4) store_state<RT, VT>(mrun, lrun, O, mine);
    __syncthreads();
    if (wave < 4) merge_state<RT, VT>(mrun, lrun, O, mine);
    __syncthreads();
    if (wave >= 1 && wave < 4) store_state<RT, VT>(mrun, lrun, O, mine);
    __syncthreads();
    if (wave != 0) return;
    for (int w = 1; w < 4; w++) merge_state<RT, VT>(mrun, lrun, O, xch + w * 64 * PER_LANE + lane);
#pragma unroll
    for (int t = 0; t < RT; t++) {
        float l = lrun[t];
        l += __shfl_xor(l, 16);
        l += __shfl_xor(l, 32);
        const int r = (rt0 + t) * 16 + j;
        if (r >= R) continue;
        const long slot = ((long)h * a.nch + chunk) * R + r;
        if (kg == 0) {
            a.part_ml[slot * 2] = mrun[t];
            a.part_ml[slot * 2 + 1] = l;
        }
        float* o = a.part_o + slot * HD + 4 * kg;
#pragma unroll
        for (int d = 0; d < VT; d++) *(float4v*)(o + 16 * d) = O[t][d];
    }
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
template <int NCH>
__global__ void k_attn_combine(AttnArgs a, int G, int R) {
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
    const _Float16 o16 = (_Float16)(num / s_den);
    const int kk = qh * hd + d;
    ((_Float16*)a.xfrag)[frag_index(kk, m)] = o16;
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
    hipLaunchKernelGGL((k_attn_partial<HD, RT, STAGES>), dim3(a.nch, a.nkv, groups), dim3(512), lds, s, a, G, R);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

template <int HD>
static int launch_hd(hipStream_t s, const AttnArgs& a0, int m, int G, int R) {
    const int trt = (R + 15) / 16;
    // more than 32 (row, q head) pairs: groups of 32 in grid z, each re-reading K and V (from L2)
    const int groups = trt <= 2 ? 1 : (trt + 1) / 2;
    // about one workgroup per compute unit: the chunk count shrinks as the row groups multiply
    // (fewer, longer chunks also mean fewer partial results for the merge to read)
    AttnArgs a = a0;
    a.nch = std::max(std::min(a0.nch, 8), std::min(a0.nch, 256 / (a0.nkv * groups)));
    int rc;
    if (trt <= 1)
        rc = launch_partial<HD, 1, 3>(s, a, G, R, 1);
    else
        rc = launch_partial<HD, 2, 3>(s, a, G, R, groups);
    if (rc) return rc;
    const dim3 cgrid(m, a.nq), cblock(HD < 64 ? 64 : HD);
    // the chunk count as a compile-time constant puts every partial's load in flight before the
    // first add (a counted loop waits on each in turn); the sum runs in the same order either way
#define TSV_COMBINE(N) \
    case N: hipLaunchKernelGGL(k_attn_combine<N>, cgrid, cblock, 0, s, a, G, R); break;
    switch (a.nch) {
        TSV_COMBINE(1) TSV_COMBINE(2) TSV_COMBINE(3) TSV_COMBINE(4) TSV_COMBINE(5) TSV_COMBINE(6) TSV_COMBINE(7) TSV_COMBINE(8)
        TSV_COMBINE(9) TSV_COMBINE(10) TSV_COMBINE(11) TSV_COMBINE(12) TSV_COMBINE(13) TSV_COMBINE(14) TSV_COMBINE(15)
        TSV_COMBINE(16) TSV_COMBINE(17) TSV_COMBINE(18) TSV_COMBINE(19) TSV_COMBINE(20) TSV_COMBINE(21) TSV_COMBINE(22)
        TSV_COMBINE(23) TSV_COMBINE(24) TSV_COMBINE(25) TSV_COMBINE(26) TSV_COMBINE(27) TSV_COMBINE(28) TSV_COMBINE(29)
        TSV_COMBINE(30) TSV_COMBINE(31) TSV_COMBINE(32)
        default: hipLaunchKernelGGL(k_attn_combine<0>, cgrid, cblock, 0, s, a, G, R); break;
    }
#undef TSV_COMBINE
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

int launch_attention(hipStream_t s, const AttnArgs& a, int m) {
    const int G = a.nq / a.nkv, R = m * G;
    if (a.hd == 128) return launch_hd<128>(s, a, m, G, R);
    if (a.hd == 64) return launch_hd<64>(s, a, m, G, R);
    set_error("attention: head_dim must be 64 or 128");
    return TSV_ERR_UNSUPPORTED;
}

}  // namespace tsv
