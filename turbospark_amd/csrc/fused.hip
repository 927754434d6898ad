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

namespace tsv {

namespace {

constexpr int XCDS = 8;
constexpr int WGS_PER_XCD = 32;
constexpr unsigned SPIN_LIMIT = 1u << 22;

struct XcdCtx {
    int xcc, rank;
    unsigned* bar;
    unsigned next_target;
    int* err;
};

// Identifies the workgroup's XCD and its rank among that XCD's workgroups.  The rank counter
// only ever grows by 32 per launch, so the low five bits are the rank.
__device__ __forceinline__ bool xcd_enter(XcdCtx& c, const FusedSync& s, int* lds_i) {
    if (threadIdx.x == 0) {
        unsigned xcc;
        asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
        xcc &= 0xFu;
        lds_i[0] = (int)xcc;
        lds_i[1] = xcc < XCDS ? (int)(__hip_atomic_fetch_add(s.rank_ctr + xcc * 64, 1u, __ATOMIC_RELAXED,
                                                            __HIP_MEMORY_SCOPE_AGENT) &
                                      (WGS_PER_XCD - 1))
                              : -1;
    }
    __syncthreads();
    c.xcc = lds_i[0];
    c.rank = lds_i[1];
    c.err = s.err;
    if (c.rank < 0) {
        if (threadIdx.x == 0) *s.err = 2;
        return false;
    }
    c.bar = s.bar_ctr + c.xcc * 64;
    c.next_target = s.bar_base + WGS_PER_XCD;
    __syncthreads();
    return true;
}

// Barrier over the 32 workgroups of this XCD.  Every wave first waits for its own stores to be
// acknowledged by the L2.
__device__ __forceinline__ bool xcd_barrier(XcdCtx& c, int* lds_i) {
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    __syncthreads();
    if (threadIdx.x == 0) {
        __hip_atomic_fetch_add(c.bar, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        unsigned n = 0;
        int ok = 1;
        while ((int)(__hip_atomic_load(c.bar, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - c.next_target) < 0) {
            if (++n > SPIN_LIMIT) {
                ok = 0;
                *c.err = 1;
                break;
            }
        }
        lds_i[2] = ok;
    }
    __syncthreads();
    c.next_target += WGS_PER_XCD;
    const bool ok = lds_i[2] != 0;
    __syncthreads();
    return ok;
}

__device__ __forceinline__ float ld_sc1(const float* base, int idx) {
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, 0x7FFFFFFF, 0x00027000);
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, idx * 4, 0, 16));
}

// ---- P0: residual add + RMSNorm inputs, spread over the XCD's workgroups ---------------------
// x[b][:] += sum of the incoming partial sums (fixed order); this XCD's private copy of the
// fp16 fragments of x * norm_w with their sub-block sums; and sum(x^2) over this workgroup's
// columns.  Every XCD computes the same numbers; XCD 0 stores x, into a second buffer because
// the other XCDs read the old rows at their own pace.
__device__ __forceinline__ void norm_inputs(const NormStage& n, const XcdCtx& c, int M, float* lds_f) {
    const int cpw = n.hidden / WGS_PER_XCD;  // columns per workgroup, a multiple of 32
    const int col0 = c.rank * cpw;
    _Float16* frag = (_Float16*)(n.frag + (size_t)c.xcc * n.frag_stride);
    float* sums = (float*)((char*)frag + xfrag_sum_offset(n.hidden));
    const int lane = threadIdx.x & 63;
    const int nslot = cpw >> 5;
    for (int idx = threadIdx.x; idx < cpw * 16; idx += 512) {
        const int b = idx / cpw, cl = idx - b * cpw, col = col0 + cl;
        float xv = 0.f;
        if (b < M) {
            xv = n.x_in[(size_t)b * n.hidden + col];
            float p[8];
#pragma unroll
            for (int s = 0; s < 8; s++) p[s] = s < n.n_partials ? n.partial[((size_t)s * 16 + b) * n.hidden + col] : 0.f;
#pragma unroll
            for (int s = 0; s < 8; s++) xv += p[s];
            if (c.xcc == 0) n.x_out[(size_t)b * n.hidden + col] = xv;
        }
        const _Float16 h = (_Float16)(xv * n.norm_w[col]);
        if (b < M) frag[frag_index(col, b)] = h;
        float sum = (float)h, sq = xv * xv;
#pragma unroll
        for (int o = 1; o < 32; o <<= 1) {
            sum += __shfl_xor(sum, o);
            sq += __shfl_xor(sq, o);
        }
        if ((lane & 31) == 0) {
            if (b < M) sums[xsum_index(col >> 5, b)] = sum;
            lds_f[b * 8 + (cl >> 5)] = sq;
        }
    }
    __syncthreads();
    if (threadIdx.x < 16) {
        float ss = 0.f;
        for (int s = 0; s < nslot; s++) ss += lds_f[threadIdx.x * 8 + s];
        n.ssq[((size_t)c.xcc * 16 + threadIdx.x) * WGS_PER_XCD + c.rank] = ss;
    }
    __syncthreads();
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
// One wave's share of a tile: chunks [c0, c0 + nc) of the weight tile row `tile` (kchunks per
// row), against the activations whose chunk index is the weight's.  `prefetch` issues the first
// two weight stages and can run before the activations exist; `run` finishes the job.
template <class F, int NG>
struct TileJob {
    Stage<F, NG> st[2];
    const uint8_t* wt;
    int c0, nc;

    __device__ __forceinline__ void prefetch(const uint8_t* w, int kchunks, int tile, int c0_, int nc_, int lane) {
        wt = w + (size_t)tile * kchunks * F::TILE_BYTES;
        c0 = c0_;
        nc = nc_;
        if (nc <= 0) return;
        __builtin_amdgcn_sched_barrier(0);
        F::load(st[0].w, wt + (size_t)c0 * F::TILE_BYTES, lane);
        F::load(st[1].w, wt + (size_t)(c0 + min(1, nc - 1)) * F::TILE_BYTES, lane);
        __builtin_amdgcn_sched_barrier(0);
    }

    __device__ __forceinline__ void run(const ActLoader<true>& x, const Consts& k, float4v (&acc)[NG], int lane) {
#pragma unroll
        for (int g = 0; g < NG; g++) acc[g] = float4v{0.f, 0.f, 0.f, 0.f};
        if (nc <= 0) return;
        __builtin_amdgcn_sched_barrier(0);
        load_x(st[0], x, c0, lane);
        load_x(st[1], x, c0 + min(1, nc - 1), lane);
        __builtin_amdgcn_sched_barrier(0);
        int c = 0;
        for (; c + 4 <= nc; c += 2) {
#pragma unroll
            for (int s = 0; s < 2; s++) {
                compute(st[s], k, acc);
                load_stage(st[s], x, wt + (size_t)(c0 + c + s + 2) * F::TILE_BYTES, c0 + c + s + 2, lane);
            }
        }
#pragma unroll
        for (int s = 0; s < 2; s++) {
            if (c + s < nc) {
                compute(st[s], k, acc);
                if (c + s + 2 < nc) load_stage(st[s], x, wt + (size_t)(c0 + c + s + 2) * F::TILE_BYTES, c0 + c + s + 2, lane);
            }
        }
        c += 2;
#pragma unroll
        for (int s = 0; s < 2; s++)
            if (c + s < nc) compute(st[s], k, acc);
    }
};

// A workgroup's eight waves work on two tiles, four K quarters each; after the fold through LDS
// wave (4 * tile_in_wg + g) owns row group g of its tile.
__device__ __forceinline__ void quarter_split(int kchunks_lo, int kchunks_n, int q, int& c0, int& nc) {
    const int per = (kchunks_n + 3) >> 2;
    c0 = kchunks_lo + min(q * per, kchunks_n);
    nc = min(per, kchunks_lo + kchunks_n - c0);
}

template <int NG>
__device__ __forceinline__ bool fold_quarters(float4v (&acc)[NG], float4v* red, int wave, int lane, float4v& v) {
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
    extern __shared__ float4v red[];
    __shared__ float s_inv[16];
    __shared__ float s_sq[16 * 8];
    __shared__ int s_i[4];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    XcdCtx ctx;
    if (!xcd_enter(ctx, a.sync, s_i)) return;
    TRACE(0);
    const int M = a.vp->m;
    Consts k;
    k.k6400 = 0x64006400u;
    k.k5400 = 0x54005400u;
    k.k64 = 0x64646464u;
    asm volatile("" : "+v"(k.k6400), "+v"(k.k5400), "+v"(k.k64));

    // gate/up tiles of this XCD: a contiguous run, two per workgroup and round
    const int gu_per = a.gu_tiles / XCDS, gu0 = ctx.xcc * gu_per;
    const int q = wave & 3, tw = wave >> 2;
    TileJob<F, NG> job;
    int c0, nc;
    quarter_split(0, a.gu_kchunks, q, c0, nc);
    {
        const int t = 2 * ctx.rank + tw;
        job.prefetch(a.w_gate_up, a.gu_kchunks, gu0 + min(t, gu_per - 1), c0, t < gu_per ? nc : 0, lane);
    }

    TRACE(1);
    norm_inputs(a.norm, ctx, M, s_sq);
    TRACE(2);
    if (!xcd_barrier(ctx, s_i)) return;
    TRACE(3);
    norm_factors(a.norm, ctx, s_inv);
    TRACE(4);

    {
        const uint8_t* fa = a.norm.frag + (size_t)ctx.xcc * a.norm.frag_stride;
        const ActLoader<true> xa(fa, fa + xfrag_sum_offset(a.norm.hidden));
        _Float16* fc = (_Float16*)a.frag_c;
        float* fc_sums = (float*)((char*)a.frag_c + xfrag_sum_offset(a.ffn));
        for (int t0 = 2 * ctx.rank; t0 < gu_per; t0 += 2 * WGS_PER_XCD) {
            const int t = t0 + tw;
            if (t0 != 2 * ctx.rank) job.prefetch(a.w_gate_up, a.gu_kchunks, gu0 + min(t, gu_per - 1), c0, t < gu_per ? nc : 0, lane);
            float4v acc[NG];
            job.run(xa, k, acc, lane);
            float4v v;
            if (fold_quarters<NG>(acc, red, wave, lane, v) && t < gu_per) {
                // lanes 0..31: gate rows, lanes 32..63: up rows of the same 32 columns
                const int g = wave & 3, col = (gu0 + t) * 32 + (lane & 31);
#pragma unroll
                for (int i = 0; i < 4; i++) {
                    const int b = 4 * g + i;
                    const float sv = v[i] * s_inv[b];
                    const float other = __shfl_xor(sv, 32);
                    const float gate = lane < 32 ? sv : other, up = lane < 32 ? other : sv;
                    const _Float16 h = (_Float16)(silu_f(gate) * up);
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
    }

    TRACE(5);
    // down projection over this XCD's K slice; its first weights are requested before the barrier
    const int dk = a.down_kchunks / XCDS, dk0 = ctx.xcc * dk;
    quarter_split(dk0, dk, q, c0, nc);
    {
        const int t = 2 * ctx.rank + tw;
        job.prefetch(a.w_down, a.down_kchunks, min(t, a.down_tiles - 1), c0, t < a.down_tiles ? nc : 0, lane);
    }
    TRACE(6);
    if (!xcd_barrier(ctx, s_i)) return;
    TRACE(7);
    {
        const ActLoader<true> xc(a.frag_c, (const char*)a.frag_c + xfrag_sum_offset(a.ffn));
        float* out = a.partial_out + (size_t)ctx.xcc * 16 * a.norm.hidden;
        for (int t0 = 2 * ctx.rank; t0 < a.down_tiles; t0 += 2 * WGS_PER_XCD) {
            const int t = t0 + tw;
            if (t0 != 2 * ctx.rank) job.prefetch(a.w_down, a.down_kchunks, min(t, a.down_tiles - 1), c0, t < a.down_tiles ? nc : 0, lane);
            float4v acc[NG];
            job.run(xc, k, acc, lane);
            float4v v;
            if (fold_quarters<NG>(acc, red, wave, lane, v) && t < a.down_tiles) {
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
    const size_t lds = (size_t)8 * NG * 1024;
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
    if (gate_up.fmt != down.fmt) return false;
    if (gate_up.n_rows != 2 * ffn || down.k != ffn || gate_up.k != hidden || down.n_rows != hidden) return false;
    if (gate_up.n_tiles % XCDS || down.kchunks % XCDS) return false;
    if (hidden % (WGS_PER_XCD * 32) || hidden > 8192) return false;
    return true;
}

int launch_ffn_block(hipStream_t s, int fmt, FfnBlockArgs& a, int m) {
    return fmt == FMT_Q4K ? launch_ffn_f<Q4K>(s, a, m) : launch_ffn_f<Q80>(s, a, m);
}

}  // namespace tsv
