// Per-XCD fused layer kernels for gfx950.
//
// An MI355X is eight XCDs of 32 compute units, each XCD with its own L2.  Handing data from one
// compute unit to another costs ~0.7 us when both sit on the same XCD (a counter in the shared
// L2) but ~3.5 us across XCDs, about as much as ending the kernel and starting the next one.  A
// decoder layer is therefore cut the way tensor parallelism cuts it across devices, with the
// XCDs as the devices: every XCD owns one eighth of the FFN columns (and, in the attention
// block, its own KV heads), so the chain
//     residual add + RMSNorm  ->  gate/up matmul + silu-mul  ->  down matmul
// runs inside one kernel with XCD-local barriers only; the down projection is row-parallel and
// leaves one partial sum per XCD, which the next kernel adds in XCD order (the reduction that
// tensor parallelism would do with an all-reduce).  Replaces, for this path, the reference's
// dispatch sequence crates/runtime/src/families/llama/dense.rs:45-120 (FFN) under the batched
// verify contract of families/qwen/batched.rs:92-456.
//
// Memory rules inside a kernel (measured on this part): plain stores followed by
// s_waitcnt vmcnt(0) and the XCD barrier are visible to sc1 ("device-coherent") loads from any
// compute unit of the same XCD; plain loads may hit a stale line in the reader's L1.  Nothing
// written here is read by another XCD before the kernel ends.
//
// Every wait is bounded: a barrier that does not complete within its spin budget raises the
// error flag and the workgroup returns, so the grid always drains.
#include "gemm_core.h"
#include "xcd_sync.h"

namespace tsv {

namespace {

// ---- P0: residual add + RMSNorm inputs, spread over the XCD's workgroups ---------------------
// x[b][:] += sum of the incoming partial sums (fixed order); this XCD's private copy of the
// fp16 fragments of x * norm_w with their sub-block sums; and sum(x^2) over this workgroup's
// columns.  Every XCD computes the same numbers; XCD 0 stores x, into a second buffer because
// the other XCDs read the old rows at their own pace.
// Called by `nw` whole waves of the workgroup (wave index wi of nw): a wave takes rows wi,
// wi + nw, ... and all of the workgroup's columns of each, so nothing is shared between waves
// and the waves that are busy prefetching weights are not involved.
__device__ __forceinline__ void norm_inputs(const NormStage& n, const XcdCtx& c, int M, int wi, int nw) {
    const int cpw = n.hidden / WGS_PER_XCD;  // columns per workgroup, a multiple of 32, at most 256
    const int col0 = c.rank * cpw;
    _Float16* frag = (_Float16*)(n.frag + (size_t)c.xcc * n.frag_stride);
    float* sums = (float*)((char*)frag + xfrag_sum_offset(n.hidden));
    const int lane = threadIdx.x & 63;
    for (int b = wi; b < M; b += nw) {
        float xin[4], wn[4], part[4][8];
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const int cl = lane + 64 * j;
            if (cl < cpw) {
                xin[j] = n.x_in[(size_t)b * n.hidden + col0 + cl];
                wn[j] = n.norm_w[col0 + cl];
#pragma unroll
                for (int s = 0; s < 8; s++)
                    if (s < n.n_partials) part[j][s] = n.partial[((size_t)s * 16 + b) * n.hidden + col0 + cl];
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
                    if (s < n.n_partials) xv += part[j][s];
                if (c.xcc == 0) n.x_out[(size_t)b * n.hidden + col] = xv;
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
        if (lane == 0) n.ssq[((size_t)c.xcc * 16 + b) * WGS_PER_XCD + c.rank] = sq;
    }
}

// Row b's 1/rms from the XCD's 32 column partials, for all 16 rows, into LDS.
__device__ __forceinline__ void norm_factors(const NormStage& n, const XcdCtx& c, float* s_inv) {
    if (threadIdx.x < 16) {
        float p[WGS_PER_XCD];
#pragma unroll
        for (int r = 0; r < WGS_PER_XCD; r++) p[r] = ld_sc1(n.ssq, (c.xcc * 16 + threadIdx.x) * WGS_PER_XCD + r);
        float ss = 0.f;
#pragma unroll
        for (int r = 0; r < WGS_PER_XCD; r++) ss += p[r];
        s_inv[threadIdx.x] = 1.0f / sqrtf(ss / (float)n.hidden + n.eps);
    }
    __syncthreads();
}

// ---- matmul items -----------------------------------------------------------------------------
// One wave's share of a tile: chunks [c0, c0 + nc) of a weight tile row, against the activations
// whose chunk index is the weight's.
struct JobDesc {
    const uint8_t* wt;  // chunk 0 of the tile row
    int c0, nc;
};

// The weights of a job can be requested long before its activations exist -- that is what keeps
// HBM busy across the barriers.  Per wave, two chunks wait in registers and two more in LDS
// (copied there by the memory pipeline); a job's last chunks are the LDS ones, the earlier ones
// stream through the two register stages.
template <class F, int NG>
struct WaveJob {
    typename F::Regs wr[2];
    XRegs<F, NG> xr[2];
    uint32_t lds0, lds1;  // LDS addresses of this wave's two tile buffers
    int lane;

    static __device__ __forceinline__ int n_lds(int nc) { return nc >= 3 ? min(2, nc - 2) : 0; }

    __device__ __forceinline__ void issue_regs(const JobDesc& j) {
        if (j.nc <= 0) return;
        __builtin_amdgcn_sched_barrier(0);
        F::load(wr[0], j.wt + (size_t)j.c0 * F::TILE_BYTES, lane);
        F::load(wr[1], j.wt + (size_t)(j.c0 + min(1, j.nc - 1)) * F::TILE_BYTES, lane);
        __builtin_amdgcn_sched_barrier(0);
    }
    __device__ __forceinline__ void issue_lds(const JobDesc& j) {
        const int nl = n_lds(j.nc);
        __builtin_amdgcn_sched_barrier(0);
        if (nl >= 1) F::load_to_lds(lds0, j.wt + (size_t)(j.c0 + j.nc - nl) * F::TILE_BYTES, lane);
        if (nl >= 2) F::load_to_lds(lds1, j.wt + (size_t)(j.c0 + j.nc - 1) * F::TILE_BYTES, lane);
        __builtin_amdgcn_sched_barrier(0);
    }

    // after_regs() runs once both register stages are free again (the next job's issue_regs)
    template <class Fn>
    __device__ __forceinline__ void run(const JobDesc& j, const ActLoader<true>& x, const Consts& k,
                                        float4v (&acc)[NG], Fn&& after_regs) {
#pragma unroll
        for (int g = 0; g < NG; g++) acc[g] = float4v{0.f, 0.f, 0.f, 0.f};
        if (j.nc <= 0) {
            after_regs();
            return;
        }
        const int nl = n_lds(j.nc), nr = j.nc - nl, c0 = j.c0;
        auto fetch = [&](int s, int c) {
            __builtin_amdgcn_sched_barrier(0);
            load_x(xr[s], x, c, lane);
            F::load(wr[s], j.wt + (size_t)c * F::TILE_BYTES, lane);
            __builtin_amdgcn_sched_barrier(0);
        };
        auto mul = [&](int s) { compute_tile<NG>(F{}, RegSrc<F>{wr[s]}, xr[s], k, acc); };
        __builtin_amdgcn_sched_barrier(0);
        load_x(xr[0], x, c0, lane);
        load_x(xr[1], x, c0 + min(1, nr - 1), lane);
        __builtin_amdgcn_sched_barrier(0);
        int c = 0;
        for (; c + 4 <= nr; c += 2) {
#pragma unroll
            for (int s = 0; s < 2; s++) {
                mul(s);
                fetch(s, c0 + c + s + 2);
            }
        }
#pragma unroll
        for (int s = 0; s < 2; s++) {
            if (c + s < nr) {
                mul(s);
                if (c + s + 2 < nr) fetch(s, c0 + c + s + 2);
            }
        }
        c += 2;
#pragma unroll
        for (int s = 0; s < 2; s++)
            if (c + s < nr) mul(s);
        // the LDS chunks: their activations first, then whatever the caller wants in flight next
        __builtin_amdgcn_sched_barrier(0);
        if (nl >= 1) load_x(xr[0], x, c0 + nr, lane);
        if (nl >= 2) load_x(xr[1], x, c0 + nr + 1, lane);
        __builtin_amdgcn_sched_barrier(0);
        after_regs();
        if (nl >= 1) compute_tile<NG>(F{}, LdsSrc<F>{lds_after(lds0, xr[0].xs[NG - 1]), lane}, xr[0], k, acc);
        if (nl >= 2) compute_tile<NG>(F{}, LdsSrc<F>{lds_after(lds1, xr[1].xs[NG - 1]), lane}, xr[1], k, acc);
    }
};

// A workgroup's eight waves work on two tiles, four K quarters each; after the fold through LDS
// wave (4 * tile_in_wg + g) owns row group g of its tile.
__device__ __forceinline__ void quarter_split(int kchunks_lo, int kchunks_n, int q, int& c0, int& nc) {
    const int per = (kchunks_n + 3) >> 2;
    c0 = kchunks_lo + min(q * per, kchunks_n);
    nc = min(per, kchunks_lo + kchunks_n - c0);
}

// `red` shares LDS with the waves' weight buffers, which every wave has finished reading
// once it arrives here.
template <int NG>
__device__ __forceinline__ bool fold_quarters(float4v (&acc)[NG], float4v* red, int wave, int lane, float4v& v) {
    __syncthreads();
#pragma unroll
    for (int g = 0; g < NG; g++) red[(wave * NG + g) * 64 + lane] = acc[g];
    __syncthreads();
    const int g = wave & 3, t4 = wave & 4;
    const bool mine = g < NG;
    if (mine) {
        v = red[((t4 + 0) * NG + g) * 64 + lane];
#pragma unroll
        for (int q = 1; q < 4; q++) v += red[((t4 + q) * NG + g) * 64 + lane];
    }
    __syncthreads();
    return mine;
}

#ifdef TSV_FUSED_TRACE
__device__ long long g_trace[64 * 16];
#define TRACE(i)                                                                                   \
    do {                                                                                           \
        if (threadIdx.x == 0 && ctx.xcc == 0) g_trace[ctx.rank * 16 + (i)] = wall_clock64();       \
    } while (0)
#else
#define TRACE(i) \
    do {         \
    } while (0)
#endif

template <class F, int NG>
__global__ __launch_bounds__(512) void k_ffn_block(FfnBlockArgs a) {
    extern __shared__ uint8_t wbuf[];  // [8 waves][2][tile bytes]; the fold buffer overlays its start
    __shared__ float s_inv[16];
    __shared__ int s_i[4];
    float4v* red = (float4v*)wbuf;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    XcdCtx ctx;
    if (!xcd_enter(ctx, a.sync, s_i)) return;
    TRACE(0);
    const int M = a.m;
    Consts k;
    k.k6400 = 0x64006400u;
    k.k5400 = 0x54005400u;
    k.k64 = 0x64646464u;
    asm volatile("" : "+v"(k.k6400), "+v"(k.k5400), "+v"(k.k64));
    WaveJob<F, NG> job;
    job.lane = lane;
    job.lds0 = __builtin_amdgcn_readfirstlane(lds_addr(wbuf) + wave * 2 * F::TILE_BYTES);
    job.lds1 = job.lds0 + F::TILE_BYTES;

    // The workgroup's eight waves work on two tiles at a time, four K quarters each.
    const int q = wave & 3, tw = wave >> 2;
    // gate/up: this XCD's tiles are a contiguous run
    const int gu_per = a.gu_tiles / XCDS, gu0 = ctx.xcc * gu_per;
    int gc0, gnc;
    quarter_split(0, a.gu_kchunks, q, gc0, gnc);
    auto gu_job = [&](int t0) {
        const int t = t0 + tw;
        return JobDesc{a.w_gate_up + (size_t)(gu0 + min(t, gu_per - 1)) * a.gu_kchunks * F::TILE_BYTES, gc0,
                       t < gu_per ? gnc : 0};
    };
    // down: every tile, this XCD's K slice
    const int dk = a.down_kchunks / XCDS;
    int dc0, dnc;
    quarter_split(ctx.xcc * dk, dk, q, dc0, dnc);
    auto down_job = [&](int t0) {
        const int t = t0 + tw;
        return JobDesc{a.w_down + (size_t)min(t, a.down_tiles - 1) * a.down_kchunks * F::TILE_BYTES, dc0,
                       t < a.down_tiles ? dnc : 0};
    };
    const int first = 2 * ctx.rank, stride = 2 * WGS_PER_XCD;

    // Waves 3 and 7 prepare the RMSNorm inputs; the others request the weights of their first
    // gate/up job at once (loads complete in issue order, so a wave's own small loads would
    // otherwise queue behind its 36 KB of weights).
    JobDesc cur = gu_job(first);
    const bool norm_wave = q == 3;
    if (norm_wave) {
        norm_inputs(a.norm, ctx, M, tw, 2);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
    }
    job.issue_regs(cur);
    job.issue_lds(cur);
    TRACE(2);
    if (!xcd_barrier(ctx, s_i, false)) return;
    TRACE(3);

    {
        const uint8_t* fa = a.norm.frag + (size_t)ctx.xcc * a.norm.frag_stride;
        const ActLoader<true> xa(fa, fa + xfrag_sum_offset(a.norm.hidden), lane);
        _Float16* fc = (_Float16*)a.frag_c;
        float* fc_sums = (float*)((char*)a.frag_c + xfrag_sum_offset(a.ffn));
        for (int t0 = first; t0 < gu_per; t0 += stride) {
            const int t = t0 + tw;
            const bool more = t0 + stride < gu_per;
            const JobDesc next = more ? gu_job(t0 + stride) : down_job(first);
            float4v acc[NG];
            job.run(cur, xa, k, acc, [&] { job.issue_regs(next); });
            float4v v;
            const bool mine = fold_quarters<NG>(acc, red, wave, lane, v);
            job.issue_lds(next);
            cur = next;
            if (t0 == first) norm_factors(a.norm, ctx, s_inv);  // everything this wave asked for has arrived by now
            if (mine && t < gu_per) {
                // lanes 0..31: gate rows, lanes 32..63: up rows of the same 32 columns
                const int g = wave & 3, col = (gu0 + t) * 32 + (lane & 31);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int b = 4 * g + i;
                    const float sv = v[i] * s_inv[b];
                    const float other = __shfl_xor(sv, 32);
                    const float gate = lane < 32 ? sv : other, up = lane < 32 ? other : sv;
                    const _Float16 h = pinned_half((_Float16)(silu_f(gate) * up));
                    float sum = (float)h;
#pragma unroll
                    for (int o = 1; o < 32; o <<= 1) sum += __shfl_xor(sum, o);
                    if (b < M && lane < 32) {
                        fc[frag_index(col, b)] = h;
                        if (lane == 0) fc_sums[xsum_index(col >> 5, b)] = sum;
                    }
                }
            }
        }
        if (first >= gu_per) {  // this workgroup had no gate/up tile: its first down job starts here
            cur = down_job(first);
            job.issue_regs(cur);
            job.issue_lds(cur);
        }
    }
    TRACE(5);
    TRACE(6);
    if (!xcd_barrier(ctx, s_i)) return;
    TRACE(7);
    {
        const ActLoader<true> xc(a.frag_c, (const char*)a.frag_c + xfrag_sum_offset(a.ffn), lane);
        float* out = a.partial_out + (size_t)ctx.xcc * 16 * a.norm.hidden;
        for (int t0 = first; t0 < a.down_tiles; t0 += stride) {
            const int t = t0 + tw;
            const bool more = t0 + stride < a.down_tiles;
            const JobDesc next = more ? down_job(t0 + stride) : JobDesc{nullptr, 0, 0};
            float4v acc[NG];
            job.run(cur, xc, k, acc, [&] { job.issue_regs(next); });
            float4v v;
            const bool mine = fold_quarters<NG>(acc, red, wave, lane, v);
            job.issue_lds(next);
            cur = next;
            if (mine && t < a.down_tiles) {
                const int g = wave & 3, n = t * 64 + lane;
                if (n < a.norm.hidden) {
#pragma unroll
                    for (int i = 0; i < 4; i++)
                        if (4 * g + i < M) out[(size_t)(4 * g + i) * a.norm.hidden + n] = v[i];
                }
            }
        }
    }
    TRACE(8);
}

template <class F, int NG>
int launch_ffn_t(hipStream_t s, FfnBlockArgs& a) {
    // An ordinary launch: the stream is in order, so the GPU is empty when the 256 workgroups
    // (one per compute unit, at most) are dispatched and all of them become resident together.
    // (A cooperative launch would guarantee that, but goes through a separate queue whose
    // hand-over costs tens of microseconds per launch.)  The bounded barrier waits are the net.
    const size_t lds = (size_t)8 * 2 * F::TILE_BYTES;  // >= the fold buffer, 8 * NG KiB
    static bool configured = false;
    if (!configured) {
        TSV_HIP(hipFuncSetAttribute((const void*)k_ffn_block<F, NG>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        configured = true;
    }
    hipLaunchKernelGGL((k_ffn_block<F, NG>), dim3(XCDS * WGS_PER_XCD), dim3(512), lds, s, a);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

template <class F>
int launch_ffn_f(hipStream_t s, FfnBlockArgs& a, int m) {
    if (m <= 4) return launch_ffn_t<F, 1>(s, a);
    if (m <= 8) return launch_ffn_t<F, 2>(s, a);
    return launch_ffn_t<F, 4>(s, a);
}

}  // namespace

int fused_ffn_barriers() { return 2; }

#ifdef TSV_FUSED_TRACE
extern "C" int tsv_fused_trace(long long* out) {
    return hipMemcpyFromSymbol(out, HIP_SYMBOL(g_trace), sizeof(long long) * 64 * 16) == hipSuccess ? 0 : 1;
}
#endif

// Shapes the FFN block kernel takes: both matrices in one format, the gate/up tiles and the
// down projection's K chunks divisible by the XCD count, hidden a multiple of 32 * 32 columns.
bool fused_ffn_supported(const TiledW& gate_up, const TiledW& down, int hidden, int ffn) {
    if (gate_up.fmt != down.fmt || (gate_up.fmt != FMT_Q4K && gate_up.fmt != FMT_Q80)) return false;
    if (gate_up.n_rows != 2 * ffn || down.k != ffn || gate_up.k != hidden || down.n_rows != hidden) return false;
    if (gate_up.n_tiles % XCDS || down.kchunks % XCDS) return false;
    if (hidden % (WGS_PER_XCD * 32) || hidden > 8192) return false;
    return true;
}

int launch_ffn_block(hipStream_t s, int fmt, FfnBlockArgs& a, int m) {
    return fmt == FMT_Q4K ? launch_ffn_f<Q4K>(s, a, m) : launch_ffn_f<Q80>(s, a, m);
}

}  // namespace tsv
