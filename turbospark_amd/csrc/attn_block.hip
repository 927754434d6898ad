// The attention half of a decoder layer as ONE kernel on gfx950, cut across the eight XCDs the way
// tensor parallelism cuts it across devices: XCD j owns KV head j and the q heads of its group.
//
//   A  residual add (the previous matmul's partial sums, fixed order) + RMSNorm inputs, every XCD
//      for itself (its own copy of the fp16 fragments of x * w and of sum(x^2): 1/rms is applied
//      where the projection's sums are complete);
//   B  the q / k / v projection of the XCD's heads, column-parallel: one workgroup per 64-row tile
//      over the whole K, bias + NeoX rotation + fp16 q / KV-cache stores in its epilogue;
//   C  split-KV attention of the XCD's KV head over the whole context, one chunk per workgroup;
//   D  the merge of the chunk partials into the fp16 activation fragments of the output projection;
//   E  the output projection, row-parallel: every output row over the XCD's K slice (its heads'
//      columns), leaving one partial sum per XCD that the next residual kernel adds in XCD order
//      (the reduction tensor parallelism would do with an all-reduce).
//
// Stages are separated by XCD-local barriers only (xcd_sync.h); nothing written here is read by
// another XCD before the kernel ends.  Replaces, for this path, the reference's dispatch sequence
// crates/runtime/src/families/llama/attn.rs:152-369 under the batched-verify contract of
// families/qwen/batched.rs:92-456 -- five launches (norm, projection, attention, merge, output
// projection) and their four kernel boundaries.
//
// A row's bits do not depend on the width of its pass: the K split of both projections, the chunk
// assignment and every fold order are functions of the model and the context length only.
#include <cstdlib>

#include "attn_core.h"
#include "gemm_core.h"
#include "xcd_sync.h"

namespace tsv {

namespace {

#ifdef TSV_FUSED_TRACE
__device__ long long g_attn_trace[32 * 16];
#define ATRACE(i)                                                                                       \
    do {                                                                                                \
        if (threadIdx.x == 0 && ctx.xcc == 0) g_attn_trace[ctx.rank * 16 + (i)] = wall_clock64();      \
    } while (0)
#else
#define ATRACE(i) \
    do {          \
    } while (0)
#endif

// ---- stage A ------------------------------------------------------------------------------------
// Workgroup `nr` of the XCD's `n_norm` norm workgroups takes hidden / n_norm columns (a multiple of
// 32, at most 256); wave w takes rows w and w + 8.
__device__ __forceinline__ void norm_stage(const AttnBlockArgs& a, int xcc, int nr, int n_norm, int M) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int cpw = a.hidden / n_norm, col0 = nr * cpw;
    _Float16* frag = (_Float16*)(a.frag + (size_t)xcc * a.frag_stride);
    float* sums = (float*)((char*)frag + xfrag_sum_offset(a.hidden));
    for (int b = wave; b < M; b += 8) {
        float xin[4], wn[4], part[4][8];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int cl = lane + 64 * j;
            if (cl < cpw) {
                xin[j] = a.x_in[(size_t)b * a.hidden + col0 + cl];
                wn[j] = a.norm_w[col0 + cl];
#pragma unroll
                for (int s = 0; s < 8; s++)
                    if (s < a.n_partials) part[j][s] = a.partial[((size_t)s * 16 + b) * a.hidden + col0 + cl];
            }
        }
        float sq = 0.f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int cl = lane + 64 * j, col = col0 + cl;
            if (cl < cpw) {  // cpw is a multiple of 32: half waves leave together
                float xv = xin[j];
#pragma unroll
                for (int s = 0; s < 8; s++)
                    if (s < a.n_partials) xv = __fadd_rn(xv, part[j][s]);
                if (a.bias_in) xv += a.bias_in[col];
                if (xcc == 0) a.x_out[(size_t)b * a.hidden + col] = xv;
                const _Float16 h = pinned_half((_Float16)(xv * wn[j]));
                frag[frag_index(col, b)] = h;
                float sum = (float)h;
#pragma unroll
                for (int o = 1; o < 32; o <<= 1) sum += __shfl_xor(sum, o);
                if ((lane & 31) == 0) sums[xsum_index(col >> 5, b)] = sum;
                sq += xv * xv;
            }
        }
#pragma unroll
        for (int o = 1; o < 64; o <<= 1) sq += __shfl_xor(sq, o);
        if (lane == 0) a.ssq[((size_t)xcc * 16 + b) * WGS_PER_XCD + nr] = sq;
    }
}

// Row b's 1/rms from the norm workgroups' column partials (fixed order): thread b < 16 asks for its
// row's partials (ssq_load) and turns them into the factor later (ssq_factor), once the matmul that
// sits between the two has used the weights that were asked for before them.
struct SsqRegs {
    float p[16];
};
__device__ __forceinline__ void ssq_load(SsqRegs& r, const AttnBlockArgs& a, int xcc, int n_norm) {
#pragma unroll
    for (int i = 0; i < 16; i++) r.p[i] = i < n_norm ? ld_sc1(a.ssq, (xcc * 16 + (threadIdx.x & 15)) * WGS_PER_XCD + i) : 0.f;
}
__device__ __forceinline__ float ssq_factor(const SsqRegs& r, const AttnBlockArgs& a) {
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < 16; i++) ss += r.p[i];
    return 1.0f / sqrtf(ss / (float)a.hidden + a.eps);
}

// ---- stage D ------------------------------------------------------------------------------------
// One wave per (row, q head of the group, 64 head dimensions): the merge of the chunk partials with
// the arithmetic of the stand-alone merge kernel (attention.metal:122-140: m* = max m_c,
// D = sum l_c e^(m_c - m*), O = sum O_c e^(m_c - m*), out = O / D; the sink joins maximum and
// denominator only), summed over the chunks in chunk order.  Lane c < nch turns chunk c's (m, l)
// into its weight; every lane then sums its own head dimension.  nch <= 32.
template <int HD>
__device__ __forceinline__ void combine_item(const AttnArgs& a, int h, int G, int R, int item, float* wl) {
    const int lane = threadIdx.x & 63;
    constexpr int SPH = HD / 64;  // items per (row, head)
    const int rh = item / SPH, sb = item - rh * SPH;  // (row, head in group) pair; half of the head
    const int mrow = rh / G, g = rh - mrow * G, qh = h * G + g;
    const int nch = a.nch, d = sb * 64 + lane;
    const __amdgpu_buffer_rsrc_t ors = __builtin_amdgcn_make_buffer_rsrc((void*)a.part_o, 0, 0x7FFFFFFF, 0x00027000);
    const __amdgpu_buffer_rsrc_t mrs = __builtin_amdgcn_make_buffer_rsrc((void*)a.part_ml, 0, 0x7FFFFFFF, 0x00027000);
    float pre[32];
#pragma unroll
    for (int c = 0; c < 32; c++) {
        const uint32_t off = (uint32_t)((((long)h * nch + min(c, nch - 1)) * R + rh) * HD + d) * 4u;
        pre[c] = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(ors, off, 0, 16));
    }
    const uint32_t moff = (uint32_t)(((long)h * nch + min(lane, nch - 1)) * R + rh) * 8u;
    const float m_in = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(mrs, moff, 0, 16));
    const float l_in = __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(mrs, moff + 4, 0, 16));
    const float mc = lane < nch ? m_in : -INFINITY, lc = lane < nch ? l_in : 0.f;
    float mx = mc;
    for (int o = 32; o > 0; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o));
    const float sink = a.sinks ? a.sinks[qh] : -INFINITY;
    mx = fmaxf(mx, sink);
    const float w = mc > -INFINITY ? __expf(mc - mx) : 0.f;
    float den = lc * w;
    for (int o = 32; o > 0; o >>= 1) den += __shfl_xor(den, o);
    if (a.sinks) den += __expf(sink - mx);
    wl[lane] = w;
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
    float num = 0.f;
#pragma unroll
    for (int c = 0; c < 32; c++)
        if (c < nch) num = fmaf(wl[c], pre[c], num);
    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // the weights are read before the next item replaces them
    const _Float16 o16 = (_Float16)(num / den);
    const int kk = qh * HD + d;
    ((_Float16*)a.xfrag)[frag_index(kk, mrow)] = o16;
    // sum of each 32-element sub-block of the output projection's input (32 neighbouring lanes)
    float sum = (float)o16;
    for (int o = 1; o < 32; o <<= 1) sum += __shfl_xor(sum, o);
    if ((lane & 31) == 0) ((float*)((char*)a.xfrag + xfrag_sum_offset(a.nq * HD)))[xsum_index(kk >> 5, mrow)] = sum;
}

template <class F, int HD, int NG>
__global__ __launch_bounds__(512) void k_attn_block(AttnBlockArgs a) {
    extern __shared__ float4v smem[];  // attention fold exchange / matmul fold
    __shared__ float s_inv[16];
    __shared__ float s_w[8 * 64];
    __shared__ int s_i[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    XcdCtx ctx;
    if (!xcd_enter(ctx, a.sync, s_i)) return;
    ATRACE(0);
    const AttnArgs& at = a.attn;
    const int M = a.m, G = at.nq / at.nkv, R = M * G, h = ctx.xcc;
    constexpr int TPH = HD / 64;  // tiles per head
    const int T = (G + 2) * TPH;   // q / k / v tiles of this XCD's heads
    const int n_norm = T <= 16 ? 16 : 8, first_norm = WGS_PER_XCD - n_norm;
    Consts k;
    k.k6400 = 0x64006400u;
    k.k5400 = 0x54005400u;
    k.k64 = 0x64646464u;
    asm volatile("" : "+v"(k.k6400), "+v"(k.k5400), "+v"(k.k64));

    // ---- A + B: norm workgroups prepare the inputs while the projection workgroups already ask
    // for their weights (which depend on nothing)
    const bool proj_wg = ctx.rank < T, norm_wg = ctx.rank >= first_norm;
    if (proj_wg) {
        const int lt = ctx.rank;
        const int tile = lt < G * TPH         ? h * G * TPH + lt
                         : lt < (G + 1) * TPH ? (at.nq + h) * TPH + (lt - G * TPH)
                                              : (at.nq + at.nkv + h) * TPH + (lt - (G + 1) * TPH);
        const int per = (a.qkv_kchunks + 7) >> 3;
        const int c0 = min(wave * per, a.qkv_kchunks), nc = min(per, a.qkv_kchunks - c0);
        const int last = max(c0 + nc - 1, 0);
        const uint8_t* wt = a.w_qkv + (size_t)tile * a.qkv_kchunks * F::TILE_BYTES;
        Stage<F, NG> st[2];
        __builtin_amdgcn_sched_barrier(0);
        F::load(st[0].w, wt + (size_t)min(c0, last) * F::TILE_BYTES, lane);
        F::load(st[1].w, wt + (size_t)min(c0 + 1, last) * F::TILE_BYTES, lane);
        __builtin_amdgcn_sched_barrier(0);
        ATRACE(1);
        if (!xcd_barrier(ctx, s_i, false)) return;
        ATRACE(2);
        SsqRegs sq;
        __builtin_amdgcn_sched_barrier(0);
        ssq_load(sq, a, ctx.xcc, n_norm);
        const uint8_t* fa = a.frag + (size_t)ctx.xcc * a.frag_stride;
        const ActLoader<true> x(fa, fa + xfrag_sum_offset(a.hidden), lane);
        __builtin_amdgcn_sched_barrier(0);
        load_x(st[0].x, x, min(c0, last), lane);
        load_x(st[1].x, x, min(c0 + 1, last), lane);
        __builtin_amdgcn_sched_barrier(0);
        float4v acc[NG];
#pragma unroll
        for (int g = 0; g < NG; g++) acc[g] = float4v{0.f, 0.f, 0.f, 0.f};
        if (nc > 0) compute(st[0], k, acc);
        if (nc > 1) compute(st[1], k, acc);
        for (int c = 2; c < nc; c++) {  // K wider than sixteen chunks
            load_stage(st[0], x, wt + (size_t)(c0 + c) * F::TILE_BYTES, c0 + c, lane);
            compute(st[0], k, acc);
        }
        // fold the waves' accumulators in wave order; wave w finishes row groups w, w + 8, ...
#pragma unroll
        for (int g = 0; g < NG; g++) smem[(wave * NG + g) * 64 + lane] = acc[g];
        if (threadIdx.x < 16) s_inv[threadIdx.x] = ssq_factor(sq, a);
        lds_barrier();
        for (int g = wave; g < NG; g += 8) {
            float4v v = smem[g * 64 + lane];
            for (int w = 1; w < 8; w++) v += smem[(w * NG + g) * 64 + lane];
#pragma unroll
            for (int i = 0; i < 4; i++) v[i] *= s_inv[4 * g + i];
            rope_epilogue(a.rope, a.vp, tile, g, v, lane, M);
        }
        ATRACE(3);
    } else {
        if (norm_wg) norm_stage(a, ctx.xcc, ctx.rank - first_norm, n_norm, M);
        ATRACE(1);
        if (!xcd_barrier(ctx, s_i, true)) return;
        ATRACE(2);
        ATRACE(3);
    }
    if (!xcd_barrier(ctx, s_i, true)) return;
    ATRACE(4);
    if (a.stages < 3) return;

    // ---- C: this XCD's KV head, chunk = rank
    if (R <= 16)
        attn_partial_body<HD, 1, 3, true>(at, G, R, ctx.rank, h, 0, (float*)smem);
    else
        attn_partial_body<HD, 2, 3, true>(at, G, R, ctx.rank, h, 0, (float*)smem);
    ATRACE(5);
    if (!xcd_barrier(ctx, s_i, true)) return;
    ATRACE(6);
    if (a.stages < 4) return;

    // ---- D: merge; items spread one wave per workgroup first
    {
        const int items = R * (HD / 64);
        for (int item = wave * WGS_PER_XCD + ctx.rank; item < items; item += 8 * WGS_PER_XCD)
            combine_item<HD>(at, h, G, R, item, s_w + wave * 64);
    }
    ATRACE(7);
    if (!xcd_barrier(ctx, s_i, true)) return;
    ATRACE(8);
    if (a.stages < 5) return;

    // ---- E: output projection over this XCD's K slice; a workgroup takes tiles rank, rank + 32, ...
    {
        const int cpx = a.wo_kchunks / XCDS;  // chunks of the XCD's slice: 1, 2, 4 or 8
        const int tpw = (a.wo_tiles + WGS_PER_XCD - 1) / WGS_PER_XCD, units = tpw * cpx;
        const ActLoader<true> x(at.xfrag, (const char*)at.xfrag + xfrag_sum_offset(at.nq * HD), lane);
        float* out = a.partial_out + (size_t)ctx.xcc * 16 * a.hidden;
        for (int u0 = 0; u0 < units; u0 += 8) {
            const int u = u0 + wave, ti = u / cpx, ck = ctx.xcc * cpx + (u - ti * cpx);
            const int tile = ctx.rank + WGS_PER_XCD * ti;
            const bool valid = u < units && tile < a.wo_tiles;
            float4v acc[NG];
#pragma unroll
            for (int g = 0; g < NG; g++) acc[g] = float4v{0.f, 0.f, 0.f, 0.f};
            if (valid) {
                Stage<F, NG> st;
                load_stage(st, x, a.w_o + ((size_t)tile * a.wo_kchunks + ck) * F::TILE_BYTES, ck, lane);
                compute(st, k, acc);
            }
            if (u0) lds_barrier();
#pragma unroll
            for (int g = 0; g < NG; g++) smem[(wave * NG + g) * 64 + lane] = acc[g];
            lds_barrier();
            const int tiles_round = 8 / cpx;
            for (int it = wave; it < tiles_round * NG; it += 8) {
                const int tt = it / NG, g = it - tt * NG, wv = tt * cpx;
                float4v v = smem[(wv * NG + g) * 64 + lane];
                for (int c = 1; c < cpx; c++) v += smem[((wv + c) * NG + g) * 64 + lane];
                const int otile = ctx.rank + WGS_PER_XCD * (u0 / cpx + tt), n = otile * 64 + lane;
                if (otile < a.wo_tiles && n < a.hidden) {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        if (4 * g + i < M) out[(size_t)(4 * g + i) * a.hidden + n] = v[i];
                }
            }
        }
    }
    ATRACE(9);
}

template <class F, int HD, int NG>
int launch_t(hipStream_t s, const AttnBlockArgs& a) {
    // LDS: the attention fold needs 4 slots x PER_LANE x 64 floats (two row tiles), the matmul folds less
    constexpr int PER_LANE = 2 * (HD / 16) * 4 + 4;
    const size_t lds = (size_t)4 * 64 * PER_LANE * 4;
    static bool configured = false;
    if (!configured) {
        TSV_HIP(hipFuncSetAttribute((const void*)k_attn_block<F, HD, NG>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        configured = true;
    }
    // An ordinary launch: the stream is in order, so the GPU is empty when the 256 workgroups (one
    // per compute unit: the LDS request allows no second one) are dispatched and all of them become
    // resident together.  The bounded barrier waits are the net.
    hipLaunchKernelGGL((k_attn_block<F, HD, NG>), dim3(XCDS * WGS_PER_XCD), dim3(512), lds, s, a);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

template <class F, int HD>
int launch_hd(hipStream_t s, const AttnBlockArgs& a) {
    return a.m <= 4 ? launch_t<F, HD, 1>(s, a) : launch_t<F, HD, 2>(s, a);
}

template <class F>
int launch_f(hipStream_t s, const AttnBlockArgs& a) {
    return a.attn.hd == 128 ? launch_hd<F, 128>(s, a) : launch_hd<F, 64>(s, a);
}

}  // namespace

int attn_block_barriers() { return 4; }

#ifdef TSV_FUSED_TRACE
extern "C" int tsv_attn_trace(long long* out) {
    return hipMemcpyFromSymbol(out, HIP_SYMBOL(g_attn_trace), sizeof(long long) * 32 * 16) == hipSuccess ? 0 : 1;
}
#endif

// Shapes the attention block takes: eight KV heads (one per XCD), at most 32 (row, q head) pairs per
// KV head, the fused q/k/v projection with the rotating epilogue, both projections in one of the
// formats below, hidden a multiple of 32 x 16 columns and at most 4096, the output projection's K
// chunks divisible by eight with a slice of 1, 2, 4 or 8 chunks per XCD.
bool attn_block_supported(const TiledW& qkv, const TiledW& wo, int hidden, int nq, int nkv, int hd, bool rope_fused) {
    if (!rope_fused || nkv != XCDS || (hd != 64 && hd != 128) || nq % nkv) return false;
    if (qkv.fmt != wo.fmt || (qkv.fmt != FMT_Q4K && qkv.fmt != FMT_Q80)) return false;
    const int G = nq / nkv, T = (G + 2) * (hd / 64);
    if (T > 16) return false;
    if (hidden % (16 * 32) || hidden > 4096 || hidden / 16 > 256) return false;
    if (qkv.k != hidden || wo.k != nq * hd || wo.n_rows != hidden) return false;
    if (wo.kchunks % XCDS) return false;
    const int cpx = wo.kchunks / XCDS;
    if (cpx != 1 && cpx != 2 && cpx != 4 && cpx != 8) return false;
    if (cpx * fmt_chunk_elems(wo.fmt) != G * hd) return false;  // the slice is exactly the XCD's heads
    return true;
}

int launch_attn_block(hipStream_t s, int fmt, const AttnBlockArgs& a) {
    if (a.m < 1 || a.m > 8 || a.m * (a.attn.nq / a.attn.nkv) > 32 || a.attn.nch != WGS_PER_XCD) {
        set_error("attention block: at most 8 rows and 32 (row, q head) pairs per KV head, 32 chunks");
        return TSV_ERR_INVALID;
    }
    return fmt == FMT_Q4K ? launch_f<Q4K>(s, a) : launch_f<Q80>(s, a);
}

}  // namespace tsv
