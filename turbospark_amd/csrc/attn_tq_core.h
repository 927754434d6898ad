// The split-KV attention pass of attn_core.h over a layer whose K / V rows are stored quantized
// (TurboQuant: crates/compute/src/kv_quant.rs:340-382, attention in the rotated space as
// crates/compute/src/kv_quant_attention.rs:58-136 does it): the workgroup reads the packed codebook
// indices and the row norms -- a quarter of the fp16 rows' bytes at four bits -- and decodes them in
// registers on the way into the same two MFMAs.
//
//   score(p)   = <q_rot, codebook_k[idx_k(p, .)]> * norm_k(p) * scale     (kv_quant_attention.rs:96-103)
//   acc_rot   += (weight(p) * norm_v(p)) * codebook_v[idx_v(p, .)]         (kv_quant_attention.rs:121-129)
//
// The codebook levels enter the MFMAs as fp16 (|level| < 1), the norms stay f32: the key norm
// multiplies the f32 score, the value norm multiplies the weight before it is rounded to fp16.  q
// arrives already rotated with the key signs; the merge kernel rotates the sum back.
//
// Store layout (one set per layer): K indices [kv head][position][HD * KB / 32 words], LSB first as
// kv_quant.rs:289-312 packs a row; V indices transposed per block of sixteen positions,
// [kv head][block][dim][group], a group holding the sixteen positions' indices of one dimension LSB
// first (32 bits at two bits per index, 64 otherwise) -- the four positions a lane feeds the second
// MFMA are then adjacent bits of one group; norms [kv head][position] f32 per side.
#pragma once
#include "attn_core.h"

namespace tsv {

template <int B>
struct TqWidth {
    static constexpr int PAIR_BITS = 2 * B, PAIR_MASK = (1 << (2 * B)) - 1;
};

// two adjacent indices -> two fp16 levels, from a table in LDS
__device__ __forceinline__ void tq_fill_pairs(uint32_t* table, const float* cb, int bits, int tid, int nthreads) {
    const int n = 1 << (2 * bits), mask = (1 << bits) - 1;
    for (int i = tid; i < n; i += nthreads) {
        const _Float16 lo = (_Float16)cb[i & mask], hi = (_Float16)cb[i >> bits];
        table[i] = (uint32_t)__builtin_bit_cast(uint16_t, lo) | ((uint32_t)__builtin_bit_cast(uint16_t, hi) << 16);
    }
}

// xch: [4 slots][PER_LANE values][64 lanes] floats of LDS; kpair / vpair: the two pair tables
template <int HD, int RT, int STAGES, int KB, int VB>
__device__ __forceinline__ void attn_partial_body_tq(const AttnArgs& a, int G, int R, int chunk, int h, int rt0, float* xch,
                                                     const uint32_t* kpair, const uint32_t* vpair) {
    constexpr int NW = 8;
    constexpr int KS = HD / 32;  // K steps of the score MFMA
    constexpr int VT = HD / 16;  // output tiles along head_dim
    constexpr int PER_LANE = RT * VT * 4 + 2 * RT;
    constexpr int KW = HD * KB / 32;            // words of a K row
    constexpr int KL = KB == 3 ? 2 : 1;         // words a lane's eight indices can touch
    constexpr int VG = tq_v_group_words(VB);    // words of a V group
    constexpr int VL = VB == 3 ? 2 : 1;         // words of it a lane loads

    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j = lane & 15, kg = lane >> 4;
    const VerifyParams* vp = a.vp;
    const int M = a.base_hint >= 0 ? a.m_hint : vp->m, base = a.base_hint >= 0 ? a.base_hint : vp->base, kvlen = base + M;
    const int nblk = (kvlen + 15) >> 4;
    const int bpc = (nblk + a.nch - 1) / a.nch;
    const int b0 = chunk * bpc, b1 = min(b0 + bpc, nblk);
    const float scale = a.scale;
    const uint32_t mmask = (1u << M) - 1u;  // slots that exist in this pass

    uint4 qf[RT][KS];
    uint32_t anc[RT];
#pragma unroll
    // lanes past the last (row, q head) pair work on pair 0 (their column is never stored): no loads under a
    // divergent branch
    for (int t = 0; t < RT; t++) {
        const int r = (rt0 + t) * 16 + j;
        const int rr = r < R ? r : 0;
        const int mrow = rr / G, g = rr - mrow * G;
        const uint32_t anc_row = vp->anc[mrow];
        const _Float16* q = (const _Float16*)a.q16 + ((long)mrow * a.nq + h * G + g) * HD + 8 * kg;
#pragma unroll
        for (int s = 0; s < KS; s++) qf[t][s] = *(const uint4*)(q + 32 * s);
        anc[t] = anc_row;
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

    // this head's stores as buffers that end after block b1 - 1 (a read past the end returns zero)
    const int cap = a.max_ctx, nbc = cap >> 4;
    const __amdgpu_buffer_rsrc_t krs = __builtin_amdgcn_make_buffer_rsrc((void*)(a.tq.kq + (long)h * cap * KW), 0, b1 * 16 * KW * 4, 0x00027000);
    const __amdgpu_buffer_rsrc_t vrs = __builtin_amdgcn_make_buffer_rsrc((void*)(a.tq.vq + (long)h * nbc * HD * VG), 0, b1 * HD * VG * 4, 0x00027000);
    const __amdgpu_buffer_rsrc_t knrs = __builtin_amdgcn_make_buffer_rsrc((void*)(a.tq.kn + (long)h * cap), 0, b1 * 64, 0x00027000);
    const __amdgpu_buffer_rsrc_t vnrs = __builtin_amdgcn_make_buffer_rsrc((void*)(a.tq.vn + (long)h * cap), 0, b1 * 64, 0x00027000);
    struct Blk {
        uint32_t kw[KS][KL];
        uint32_t vw[VT][VL];
        u32x4 kn, vn;
    };
    // the lane's eight K indices of score step s start at bit (32 s + 8 kg) * KB of its row
    uint32_t kwoff[KS], ksh[KS];
#pragma unroll
    for (int s = 0; s < KS; s++) {
        const uint32_t bit = (uint32_t)(32 * s + 8 * kg) * KB;
        kwoff[s] = ((uint32_t)j * KW + (bit >> 5)) * 4;
        ksh[s] = bit & 31;
    }
    // its four V indices of output tile d are bits 4 kg VB .. of the group of dimension 16 d + j
    const uint32_t vbit = (uint32_t)(4 * kg) * VB;
    const uint32_t vwoff = ((uint32_t)j * VG + (VB == 4 ? (vbit >> 5) : 0)) * 4, vsh = VB == 4 ? (vbit & 31) : vbit;
    const int nb = b1 > b0 + wave ? (b1 - b0 - wave + NW - 1) / NW : 0;  // blocks of this wave
    auto fetch = [&](Blk& st, int i) {
        const int blk = b0 + wave + NW * i;
        const uint32_t ko = (uint32_t)blk * (16 * KW * 4), vo = (uint32_t)blk * (HD * VG * 4), no = (uint32_t)blk * 64 + 16 * kg;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < KS; s++)
#pragma unroll
            for (int l = 0; l < KL; l++) st.kw[s][l] = __builtin_amdgcn_raw_buffer_load_b32(krs, ko + kwoff[s] + 4 * l, 0, 0);
#pragma unroll
        for (int d = 0; d < VT; d++)
#pragma unroll
            for (int l = 0; l < VL; l++)
                st.vw[d][l] = __builtin_amdgcn_raw_buffer_load_b32(vrs, vo + vwoff + (uint32_t)d * (16 * VG * 4) + 4 * l, 0, 0);
        st.kn = __builtin_amdgcn_raw_buffer_load_b128(knrs, no, 0, 0);
        st.vn = __builtin_amdgcn_raw_buffer_load_b128(vnrs, no, 0, 0);
        __builtin_amdgcn_sched_barrier(0);
    };
    auto consume = [&](const Blk& st, int i) {
        const int p0 = (b0 + wave + NW * i) << 4;
        const bool tail = p0 + 16 > base;
        // the block's K levels as the score MFMA's fragments
        u32x4 kf[KS];
#pragma unroll
        for (int s = 0; s < KS; s++) {
            const uint32_t field = KL == 2 ? __builtin_amdgcn_alignbit(st.kw[s][KL - 1], st.kw[s][0], ksh[s]) : st.kw[s][0] >> ksh[s];
#pragma unroll
            for (int e = 0; e < 4; e++) kf[s][e] = kpair[(field >> (TqWidth<KB>::PAIR_BITS * e)) & TqWidth<KB>::PAIR_MASK];
        }
        // the norms as scalars (a bit cast applied to a vector element in place reads element 0 whatever the index)
        const uint32_t knb[4] = {st.kn[0], st.kn[1], st.kn[2], st.kn[3]}, vnb[4] = {st.vn[0], st.vn[1], st.vn[2], st.vn[3]};
        u32x2 vf[VT];
#pragma unroll
        for (int d = 0; d < VT; d++) {
            const uint32_t quad = VL == 2 ? (uint32_t)((((uint64_t)st.vw[d][VL - 1] << 32) | st.vw[d][0]) >> vsh) : st.vw[d][0] >> vsh;
            vf[d][0] = vpair[quad & TqWidth<VB>::PAIR_MASK];
            vf[d][1] = vpair[(quad >> TqWidth<VB>::PAIR_BITS) & TqWidth<VB>::PAIR_MASK];
        }
#pragma unroll
        for (int t = 0; t < RT; t++) {
            float4v S = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < KS; s++)
                S = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, kf[s]), __builtin_bit_cast(half8, qf[t][s]), S,
                                                           0, 0, 0);
            uint32_t vis4 = 0xFu;
            if (tail) {
                const uint64_t w = ((uint64_t)(anc[t] & mmask) << 16) | 0xFFFFull;
                vis4 = (uint32_t)(w >> (p0 + 4 * kg - base + 16)) & 0xFu;  // shift in [1, 47]
            }
            float sc[4];
#pragma unroll
            for (int i4 = 0; i4 < 4; i4++)
                sc[i4] = ((vis4 >> i4) & 1u) ? (S[i4] * __uint_as_float(knb[i4])) * scale : -INFINITY;
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
                    ps += p;  // the denominator takes the weight alone, the value norm rides with the numerator
                    P[i4] = (_Float16)(p * __uint_as_float(vnb[i4]));
                }
                lrun[t] = fmaf(lrun[t], alpha, ps);
                mrun[t] = mnew;
            }
            // once the running maximum has settled the factor is exactly 1 in every lane: the products are
            // skipped then (the same bits), which is most blocks of a long context
            if (__builtin_amdgcn_ballot_w64(alpha != 1.f) != 0) {
#pragma unroll
                for (int d = 0; d < VT; d++) O[t][d] *= alpha;
            }
#pragma unroll
            for (int d = 0; d < VT; d++) {
                O[t][d] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4, vf[d]), P, O[t][d], 0, 0, 0);
            }
        }
    };
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

}  // namespace tsv
