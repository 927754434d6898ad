// Device-side core of the split-KV GQA attention of a verify pass: one workgroup's pass over its
// chunk of the context (crates/gpu/src/attention_decode.rs:1092-1363; arithmetic contract
// crates/compute/src/attention.rs:53-137).  Shared by the stand-alone attention kernel and the
// per-XCD fused attention block.
#pragma once
#include <type_traits>

#include "tsv_internal.h"

namespace tsv {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// The library is compiled with -ffp-contract=off and every fused multiply-add here is written out:
// left to itself the compiler contracts a * b + c * d one way in one template instantiation and the
// other way in the next, and a row's bits would then depend on how many rows share its pass.
//
// One (m, l, O) running state merged into another (flash-decoding rescale).
// (BASE2: the maxima are kept in units of log 2, the weights are powers of two)
template <int RT, int VT, bool BASE2 = false>
__device__ __forceinline__ void merge_state(float (&mrun)[RT], float (&lrun)[RT], float4v (&O)[RT][VT], const float* src) {
    // `src` points at this lane's column of a [values][64 lanes] slot: consecutive lanes touch
    // consecutive LDS banks
#pragma unroll
    for (int t = 0; t < RT; t++) {
        const float m1 = src[64 * (2 * t)], l1 = src[64 * (2 * t + 1)];
        const float mnew = fmaxf(mrun[t], m1);
        if (mnew > -INFINITY) {
            const float a0 = BASE2 ? __builtin_amdgcn_exp2f(mrun[t] - mnew) : __expf(mrun[t] - mnew);
            const float a1 = BASE2 ? __builtin_amdgcn_exp2f(m1 - mnew) : __expf(m1 - mnew);
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

// max over the four lanes l, l ^ 16, l ^ 32, l ^ 48 (the four position groups of one (row, q head) pair), in every
// one of them, on the vector ALU: v_permlane16_swap exchanges the odd 16-lane rows of its first operand with the even
// rows of its second, v_permlane32_swap the upper half of the first with the lower half of the second, so with the
// same value in both operands the two results hold the value of lane l and of its partner.  (Written as assembly:
// the compiler folds max(result 0, result 1) of the builtin with equal operands into result 0.)
__device__ __forceinline__ float max4(float a, float b, float c, float d) {
    float r;
    asm("v_max_f32 %0, %1, %2\n\tv_max3_f32 %0, %0, %3, %4" : "=&v"(r) : "v"(a), "v"(b), "v"(c), "v"(d));
    return r;
}
constexpr float REF_SLACK = 8.0f;
__device__ __forceinline__ float max_over_position_groups(float v) {
    float w = v;
    asm volatile("s_nop 1\n\tv_permlane16_swap_b32 %0, %1\n\tv_max_f32 %0, %0, %1" : "+v"(v), "+v"(w));
    w = v;
    asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\tv_max_f32 %0, %0, %1" : "+v"(v), "+v"(w));
    return v;
}

// The waves of a workgroup share a chunk of the context.  A pass of more than RT row tiles is split into TG tile
// groups: wave w works on group w % TG (row tiles RT * group ..) and walks every NW-th 16-position block of the
// chunk, NW = attn_phases(TG), starting at block w / TG, with up to STAGES blocks of K and V in flight.  The waves of
// different groups that walk the same blocks run side by side on one compute unit, so a block comes out of the L2
// once for all (row, q head) pairs of the pass.  (Legacy callers pass TG = 1 and their own rt0: eight waves, one group.)
// COH: the query rows and the K / V blocks are read device-coherently (sc1), for a caller whose
// other compute units wrote them earlier in the same kernel.
// xch: [TG][min(NW, 4) slots][PER_LANE values][64 lanes] floats of LDS.
__host__ __device__ constexpr int attn_phases(int tg) { return tg == 1 ? 8 : tg == 2 ? 4 : 2; }

template <int HD, int RT, int STAGES, bool COH, int TG = 1>
__device__ __forceinline__ void attn_partial_body(const AttnArgs& a, int G, int R, int chunk, int h, int rt_first, float* xch) {
    constexpr int NW = attn_phases(TG);
    constexpr int KS = HD / 32;  // K steps of the score MFMA
    constexpr int VT = HD / 16;  // output tiles along head_dim
    constexpr int PER_LANE = RT * VT * 4 + 2 * RT;
    constexpr int POLICY = COH ? 16 : 0;  // buffer-load cache policy: sc1

    // (the wave index as a scalar: everything derived from it -- block numbers, the choice of variant -- then stays
    // on the scalar unit)
    const int lane = threadIdx.x & 63, wave_in_wg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int tg = TG == 1 ? 0 : wave_in_wg % TG, wave = TG == 1 ? wave_in_wg : wave_in_wg / TG;  // wave: the phase
    const int rt0 = rt_first + tg * RT;
    const int j = lane & 15, kg = lane >> 4;
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
    int lo[RT];  // the row's position: with a window it sees positions lo + 1 - window .. lo
#pragma unroll
    // Lanes past the last (row, q head) pair work on pair 0 (a column of the MFMAs of their own, never stored):
    // loads under a divergent branch would be waited for, all of them, where the branches join -- a memory round
    // trip per row tile before the first K / V load is even issued.
    for (int t = 0; t < RT; t++) {
        const int r = (rt0 + t) * 16 + j;
        const int rr = r < R ? r : 0;
        const int mrow = rr / G, g = rr - mrow * G;
        const uint32_t anc_row = vp->anc[mrow];
        const int pos_row = vp->pos[mrow];
        const _Float16* q = (const _Float16*)a.q16 + ((long)mrow * a.nq + h * G + g) * HD + 8 * kg;
        if (COH) {
            const __amdgpu_buffer_rsrc_t qrs = __builtin_amdgcn_make_buffer_rsrc((void*)a.q16, 0, 0x7FFFFFFF, 0x00027000);
            const uint32_t qo = (uint32_t)((const char*)q - (const char*)a.q16);
#pragma unroll
            for (int s = 0; s < KS; s++)
                qf[t][s] = __builtin_bit_cast(uint4, __builtin_amdgcn_raw_buffer_load_b128(qrs, qo + 64 * s, 0, 16));
        } else {
#pragma unroll
            for (int s = 0; s < KS; s++) qf[t][s] = *(const uint4*)(q + 32 * s);
        }
        // taken as loaded (for a lane past the end: pair 0's), and not touched before the first K / V loads are out
        anc[t] = anc_row;
        lo[t] = pos_row;
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

    // this head's K and V blocks (kcache_index / vcache_index: a block is KS, resp. VT / 2, runs of one KiB, each
    // what one wave-wide 16-byte load takes) as buffers that end after block b1 - 1; a ring layer
    // (kv_cache.rs:360-378: position p lives in slot p % capacity) keeps block b in slot b % nbc
    const bool ring = a.ring != 0;
    const int nbc = a.max_ctx >> 4;
    const uint32_t blk_bytes = 16 * HD * 2;
    const __amdgpu_buffer_rsrc_t krs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)((const _Float16*)a.kc + (long)h * (a.max_ctx >> 4) * (HD * 16)), 0, (int)((ring ? nbc : b1) * blk_bytes), 0x00027000);
    const __amdgpu_buffer_rsrc_t vrs = __builtin_amdgcn_make_buffer_rsrc(
        (void*)((const _Float16*)a.vc + (long)h * (a.max_ctx >> 4) * (HD * 16)), 0, (int)((ring ? nbc : b1) * blk_bytes), 0x00027000);
    struct Blk {
        u32x4 kf[KS];
        u32x4 vf[VT / 2];  // two output tiles' operands per load
    };
    const uint32_t loff = (uint32_t)lane * 16;
    const int nb = b1 > b0 + wave ? (b1 - b0 - wave + NW - 1) / NW : 0;  // blocks of this wave
    auto fetch = [&](Blk& st, int i) {  // block i of this wave's run
        const int blk = b0 + wave + NW * i;
        const uint32_t bo = (uint32_t)(ring ? blk % nbc : blk) * blk_bytes;
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s = 0; s < KS; s++) st.kf[s] = __builtin_amdgcn_raw_buffer_load_b128(krs, bo + loff + 1024 * s, 0, POLICY);
#pragma unroll
        for (int u = 0; u < VT / 2; u++) st.vf[u] = __builtin_amdgcn_raw_buffer_load_b128(vrs, bo + loff + 1024 * u, 0, POLICY);
        __builtin_amdgcn_sched_barrier(0);
    };
    // Scores are kept in units of log 2 (one multiply by scale * log2(e), then v_exp_f32 as it is), and a block that
    // lies wholly inside the committed prefix and inside every row's window -- nearly all of a long context -- takes
    // the variant without the visibility words (a wave-uniform choice; a visible position gets the same operations
    // in the same order in both, so its bits do not depend on which variant its block took).
    const float c2 = scale * 1.44269504088896340736f;
    auto consume = [&](const Blk& st, int i) {
        const int p0 = (b0 + wave + NW * i) << 4;
        const bool tail = p0 + 16 > base;
        // Three phases over the row tiles -- all score products, then the softmax steps, then all value products --
        // so that the matrix pipe works through one tile's chain while the vector ALU is busy with another's.
        float4v Sx[RT];
        half4 Px[RT];
#pragma unroll
        for (int t = 0; t < RT; t++) Sx[t] = float4v{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int s = 0; s < KS; s++)
#pragma unroll
            for (int t = 0; t < RT; t++)
                Sx[t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, st.kf[s]),
                                                               __builtin_bit_cast(half8, qf[t][s]), Sx[t], 0, 0, 0);
#pragma unroll
        for (int t = 0; t < RT; t++) {
            const float4v S = Sx[t];
            // (raw scores; they are scaled where they are used: the block maximum once, the weights by one fused
            // multiply-add each -- exp2(S * c2 - reference))
            float sc[4] = {S[0], S[1], S[2], S[3]};
            if (tail || p0 < cut_end) {  // (wave-uniform: a scalar branch)
                // Visibility of this lane's four positions as a 4-bit word, computed without
                // branches: bit (slot + 16) of `w` says whether cache slot base+slot is visible
                // (the 16 low bits stand for prefix positions, always visible).
                uint32_t vis4 = 0xFu;
                if (tail) {
                    const uint64_t w = ((uint64_t)(anc[t] & mmask) << 16) | 0xFFFFull;
                    vis4 = (uint32_t)(w >> (p0 + 4 * kg - base + 16)) & 0xFu;  // shift in [1, 47]
                }
                if (p0 < cut_end) {  // some row's window starts inside or after this block
                    const int d = lo[t] + 1 - window - (p0 + 4 * kg);  // this lane's positions below index d are outside
                    vis4 &= d <= 0 ? 0xFu : d >= 4 ? 0u : (0xFu << d) & 0xFu;
                }
#pragma unroll
                for (int i4 = 0; i4 < 4; i4++) sc[i4] = ((vis4 >> i4) & 1u) ? sc[i4] : -INFINITY;
            }
            const float mb = max_over_position_groups(max4(sc[0], sc[1], sc[2], sc[3])) * c2;
            // The reference the weights are taken against follows the row's maximum lazily: it moves only when the
            // block's maximum passes it by more than REF_SLACK (in units of log 2), so a weight never exceeds
            // 2^REF_SLACK -- far inside fp16 -- and the running sums are rescaled a handful of times per row instead of
            // at every new maximum (a wave that walks eight blocks of random scores would otherwise rescale in nearly
            // every one of them).  Any reference gives the same quotient; the decision is per row, from the row's own
            // scores, so a row's bits do not depend on what shares its pass.
            const bool grow = mb > mrun[t] + REF_SLACK;
            if (__builtin_amdgcn_ballot_w64(grow) != 0) {
                // a row that has seen nothing yet and sees nothing here (every position masked) keeps mrun = -inf:
                // its factor is taken against a finite stand-in and comes out as zero, on empty sums
                const float mnew = grow ? mb : mrun[t];
                const float alpha = __builtin_amdgcn_exp2f(mrun[t] - fmaxf(mnew, -3.0e38f));  // exactly 1 where the row kept its reference
                lrun[t] *= alpha;
#pragma unroll
                for (int d = 0; d < VT; d++) O[t][d] *= alpha;
                mrun[t] = mnew;
            }
            const float nref = -fmaxf(mrun[t], -3.0e38f);
            half4 P;
            float ps = 0.f;
#pragma unroll
            for (int i4 = 0; i4 < 4; i4++) {
                const float p = __builtin_amdgcn_exp2f(fmaf(sc[i4], c2, nref));
                ps += p;
                P[i4] = (_Float16)p;
            }
            lrun[t] += ps;
            Px[t] = P;
        }
#pragma unroll
        for (int d = 0; d < VT; d++) {
            const u32x4 v2 = st.vf[d >> 1];
            const u32x2 vd = (d & 1) ? u32x2{v2.z, v2.w} : u32x2{v2.x, v2.y};
#pragma unroll
            for (int t = 0; t < RT; t++)
                O[t][d] = __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(half4, vd), Px[t], O[t][d], 0, 0, 0);
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

    // fold the group's running (m, l, O): with eight phases 4..7 into 0..3 first, then 1.. into 0
    constexpr int SLOTS = NW < 4 ? NW : 4;
    float* grp = xch + tg * SLOTS * 64 * PER_LANE + lane;
    if (NW == 8) {
        if (wave >= 4) store_state<RT, VT>(mrun, lrun, O, grp + (wave & 3) * 64 * PER_LANE);
        __syncthreads();
        if (wave < 4) merge_state<RT, VT, true>(mrun, lrun, O, grp + wave * 64 * PER_LANE);
        __syncthreads();
    }
    if (wave >= 1 && wave < 4) store_state<RT, VT>(mrun, lrun, O, grp + wave * 64 * PER_LANE);
    __syncthreads();
    if (wave != 0) return;
    for (int w = 1; w < SLOTS; w++) merge_state<RT, VT, true>(mrun, lrun, O, grp + w * 64 * PER_LANE);
#pragma unroll
    for (int t = 0; t < RT; t++) {
        float l = lrun[t];
        l += __shfl_xor(l, 16);
        l += __shfl_xor(l, 32);
        const int r = (rt0 + t) * 16 + j;
        if (r >= R) continue;
        const long slot = ((long)h * a.nch + chunk) * R + r;
        if (kg == 0) {
            a.part_ml[slot * 2] = mrun[t] * 0.69314718055994530942f;  // the merge works with natural logarithms
            a.part_ml[slot * 2 + 1] = l;
        }
        float* o = a.part_o + slot * HD + 4 * kg;
#pragma unroll
        for (int d = 0; d < VT; d++) *(float4v*)(o + 16 * d) = O[t][d];
    }
}

}  // namespace tsv
