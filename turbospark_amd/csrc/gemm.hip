// Dequant-fused small-M matmul for GGUF Q4_K / Q8_0 weights on gfx950 (wave64, MFMA).
//
// Replaces the reference's batched verify GEMM (crates/gpu/src/shaders/dequant_kquant_batch.metal:62-123,
// host wrapper dequant_kquant_gemm_batch.rs:96-126): Y[b][n] = sum_k W[n][k] * X[b][k], b < 16,
// every weight byte read once for all rows.  The arithmetic contract is the CPU reference's
// (crates/compute/src/quant_gguf/q4_k.rs:67-108,207-220; q8_0.rs:19-47,80-93).
//
// How it maps to the hardware:
//  * one wave owns a 64-row tile -- lane l holds weight row l -- and walks K.  The MACs run on
//    v_mfma_f32_4x4x4_16B_f16: its 16 independent 4x4x4 blocks take four K values of four weight
//    rows each as the B operand (so all 64 lanes carry useful weights, however few activation
//    rows there are) and, through the A-broadcast control (cbsz = 4, abid = step), all share one
//    block of the A operand: four activation rows x the same four K values.  One 8-byte
//    activation load per lane therefore feeds 16 consecutive MFMAs (abid = 0..15), and a pass
//    of m rows costs ceil(m/4) MFMAs per four K values;
//  * quant codes go to the MFMA as exact fp16 integers: (v & 0x000F000F) | 0x64006400 is the
//    pair (1024+q, 1024+q'), (v & 0x00F000F0) | 0x54005400 is (64+q, 64+q') -- one
//    v_and_or_b32 per two weights, no int->float convert; the offset is removed in fp32 through
//    the per-sub-block activation sums that the Q4_K min term needs anyway:
//        y += d*sc_j * D_j - (d*sc_j*off + dmin*m_j) * sum_k x_k
//    and that part rides v_mfma_f32_4x4x1_16B_f32 (sub-block index as the broadcast selector);
//  * the element order inside a 4-wide K step is whatever the unpack produces ([0,2,1,3]); the
//    activations are stored pre-permuted instead of shuffling weights;
//  * weights are re-tiled once at load so each wave-wide load is 1 KiB contiguous (16 B per
//    lane); activations come pre-arranged as MFMA operands (512 B contiguous per load) from L2;
//  * a workgroup is `kparts` waves working on the same tile, each on its own run of K chunks,
//    whose accumulators are folded through LDS in wave order (deterministic); split-K across
//    workgroups writes partial sums that the consumer kernel adds, again in fixed order.
//    Neither split depends on the number of activation rows, so a row's result is the same
//    bits whether it is verified alone or in a block.
#include <algorithm>
#include <utility>

#include "tsv_internal.h"

namespace tsv {

typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// ------------------------------------------------------------------------------- re-tiling
// One thread per 16-byte unit of a source row's chunk (unit 8 = the scale header).
__global__ void k_repack_q4k(const uint8_t* __restrict__ raw, int n_rows, int kchunks,
                             uint8_t* __restrict__ tiles, int grp, int stride, int offset) {
    const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long total = (long)n_rows * kchunks * 9;
    if (gid >= total) return;
    const int u = (int)(gid % 9);
    const long t = gid / 9;
    const int c = (int)(t % kchunks);
    const int r = (int)(t / kchunks);
    const int drow = (r / grp) * stride + offset + r % grp;
    const int tile = drow >> 6, lane = drow & 63;
    const uint8_t* blk = raw + ((long)r * kchunks + c) * 144;
    uint8_t* dst = tiles + ((long)tile * kchunks + c) * 9216 + (u < 8 ? (u * 64 + lane) * 16 : 8192 + lane * 16);
    *(uint4*)dst = *(const uint4*)(u < 8 ? blk + 16 + 16 * u : blk);
}

__global__ void k_repack_q80(const uint8_t* __restrict__ raw, int n_rows, int kchunks,
                             uint8_t* __restrict__ tiles, int grp, int stride, int offset) {
    const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long total = (long)n_rows * kchunks * 9;
    if (gid >= total) return;
    const int u = (int)(gid % 9);
    const long t = gid / 9;
    const int c = (int)(t % kchunks);
    const int r = (int)(t / kchunks);
    const int drow = (r / grp) * stride + offset + r % grp;
    const int tile = drow >> 6, lane = drow & 63;
    const uint8_t* row = raw + (long)r * kchunks * 4 * 34 + (long)c * 4 * 34;
    uint8_t* tb = tiles + ((long)tile * kchunks + c) * 8704;
    if (u < 8) {
        const uint8_t* src = row + (u >> 1) * 34 + 2 + 16 * (u & 1);
        uint8_t* dst = tb + (u * 64 + lane) * 16;
#pragma unroll
        for (int i = 0; i < 16; i++) dst[i] = src[i];
    } else {
        uint8_t* dst = tb + 8192 + lane * 8;
#pragma unroll
        for (int b = 0; b < 4; b++) {
            dst[2 * b] = row[b * 34];
            dst[2 * b + 1] = row[b * 34 + 1];
        }
    }
}

int launch_repack(hipStream_t s, int fmt, const uint8_t* raw, int n_rows, int k, uint8_t* tiles,
                  int kchunks, int grp, int stride, int offset) {
    (void)k;
    const long total = (long)n_rows * kchunks * 9;
    if (total == 0) return TSV_OK;
    if (fmt == FMT_Q4K)
        hipLaunchKernelGGL(k_repack_q4k, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, raw, n_rows,
                           kchunks, tiles, grp, stride, offset);
    else
        hipLaunchKernelGGL(k_repack_q80, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, raw, n_rows,
                           kchunks, tiles, grp, stride, offset);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

// ------------------------------------------------------------------------------- helpers
template <int... I, class Fn>
__device__ __forceinline__ void static_for_impl(std::integer_sequence<int, I...>, Fn&& f) {
    (f(std::integral_constant<int, I>{}), ...);
}
template <int N, class Fn>
__device__ __forceinline__ void static_for(Fn&& f) {
    static_for_impl(std::make_integer_sequence<int, N>{}, f);
}

// D[i] += sum_k A_step[i][k] * B_lane[k]: A taken from block `STEP` of the a operand for all lanes
template <int STEP>
__device__ __forceinline__ float4v mfma_f16(u32x2 a, u32x2 b, float4v c) {
    return __builtin_amdgcn_mfma_f32_4x4x4f16(__builtin_bit_cast(half4, a), __builtin_bit_cast(half4, b), c, 4, STEP, 0);
}
template <int STEP>
__device__ __forceinline__ float4v mfma_f32(float a, float b, float4v c) {
    return __builtin_amdgcn_mfma_f32_4x4x1f32(a, b, c, 4, STEP, 0);
}

__device__ __forceinline__ float h2f_lo(uint32_t v) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(v & 0xFFFF));
}
__device__ __forceinline__ float h2f_hi(uint32_t v) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(v >> 16));
}
__device__ __forceinline__ float ubyte(uint32_t v, int i) { return (float)((v >> (8 * i)) & 0xFF); }

// (v & mask) | bits as ONE v_and_or_b32: the instruction can take a single literal / scalar
// operand, so the second constant is pinned in a vector register.
__device__ __forceinline__ uint32_t and_or(uint32_t v, uint32_t mask, uint32_t bits_vgpr) {
    return (v & mask) | bits_vgpr;
}

struct Consts {
    uint32_t k6400, k5400, k64;
};

// ------------------------------------------------------------------------------- formats
struct Q4K {
    static constexpr int NSUB = 8, NPAIR = 4, TILE_BYTES = 9216;
    struct Regs {
        u32x4 q[8];
        u32x4 s;
    };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* tile, int lane) {
        const u32x4* p = (const u32x4*)tile + lane;
#pragma unroll
        for (int u = 0; u < 8; u++) r.q[u] = __builtin_nontemporal_load(p + u * 64);
        r.s = __builtin_nontemporal_load(p + 512);
    }
    // float index of this lane's sub-block sums for row group g of chunk c
    static __device__ __forceinline__ int xs_index(int c, int g, int lane) { return (c * 4 + g) * 32 + (lane & 31); }
};

struct Q80 {
    static constexpr int NSUB = 4, NPAIR = 2, TILE_BYTES = 8704;
    struct Regs {
        u32x4 q[8];
        u32x2 s;
    };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* tile, int lane) {
        const u32x4* p = (const u32x4*)tile + lane;
#pragma unroll
        for (int u = 0; u < 8; u++) r.q[u] = __builtin_nontemporal_load(p + u * 64);
        r.s = __builtin_nontemporal_load((const u32x2*)(tile + 8192) + lane);
    }
    // a 128-element chunk is half of a 256-element sum group: its four sub-blocks go to blocks 0..3
    static __device__ __forceinline__ int xs_index(int c, int g, int lane) {
        return ((c >> 1) * 4 + g) * 32 + (c & 1) * 16 + (lane & 15);
    }
};

template <class F, int NG>
struct Stage {
    typename F::Regs w;
    u32x2 xa[F::NPAIR][NG];
    float xs[NG];
};

template <class F, int NG>
__device__ __forceinline__ void load_stage(Stage<F, NG>& st, const GemmArgs& a, const uint8_t* wt, int c, int lane) {
    // The loads of one stage stay together and in program order (scheduling fences on both
    // sides), so "stage s has landed" is one s_waitcnt vmcnt(n) with the same n on every path.
    __builtin_amdgcn_sched_barrier(0);
    const u32x2* xp = (const u32x2*)a.xfrag + (size_t)c * F::NPAIR * 256 + lane;
#pragma unroll
    for (int p = 0; p < F::NPAIR; p++)
#pragma unroll
        for (int g = 0; g < NG; g++) st.xa[p][g] = xp[(p * 4 + g) * 64];
#pragma unroll
    for (int g = 0; g < NG; g++) st.xs[g] = a.xsum[F::xs_index(c, g, lane)];
    F::load(st.w, wt + (size_t)c * F::TILE_BYTES, lane);
    __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ void fma4(float4v& t, float s, const float4v& d) {
    t.x = __builtin_fmaf(s, d.x, t.x);
    t.y = __builtin_fmaf(s, d.y, t.y);
    t.z = __builtin_fmaf(s, d.z, t.z);
    t.w = __builtin_fmaf(s, d.w, t.w);
}

// One Q4_K superblock tile (64 weight rows x 256 K) against NG groups of four activation rows.
//   t  = - sum_j (d*sc_j*off_j + dmin*m_j) * sum_k X_jk       8 fp32 MFMAs per group
//   t += sum_j d*sc_j * (X_j . (off_j + q_j))                  64 fp16 MFMAs per group
// Both parts are summed per tile first so the large code offsets cancel before they reach the
// running accumulator.
template <int NG>
__device__ __forceinline__ void compute(const Stage<Q4K, NG>& st, const Consts& k, float4v (&acc)[NG]) {
    const Q4K::Regs& r = st.w;
    const float d = h2f_lo(r.s.x), dmin = h2f_hi(r.s.x);
    // 6-bit scale / min unpack (q4_k.rs:43-54), four sub-blocks per 32-bit word
    const uint32_t sl = r.s.y & 0x3F3F3F3Fu, ml = r.s.z & 0x3F3F3F3Fu;
    const uint32_t sh = (r.s.w & 0x0F0F0F0Fu) | ((r.s.y >> 2) & 0x30303030u);
    const uint32_t mh = ((r.s.w >> 4) & 0x0F0F0F0Fu) | ((r.s.z >> 2) & 0x30303030u);
    float sc[8], cf[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        sc[j] = d * ubyte(j < 4 ? sl : sh, j & 3);
        const float mn = dmin * ubyte(j < 4 ? ml : mh, j & 3);
        // even sub-blocks carry the 1024 code offset, odd ones 64
        cf[j] = -__builtin_fmaf(sc[j], (j & 1) ? 64.0f : 1024.0f, mn);
    }
    float4v t[NG];
#pragma unroll
    for (int g = 0; g < NG; g++) t[g] = float4v{0.f, 0.f, 0.f, 0.f};
    static_for<8>([&](auto J) {
        constexpr int j = decltype(J)::value;
#pragma unroll
        for (int g = 0; g < NG; g++) t[g] = mfma_f32<j>(st.xs[g], cf[j], t[g]);
    });
#pragma unroll
    for (int p = 0; p < 4; p++) {
        float4v dlo[NG], dhi[NG];
#pragma unroll
        for (int g = 0; g < NG; g++) dlo[g] = dhi[g] = float4v{0.f, 0.f, 0.f, 0.f};
        static_for<8>([&](auto W) {
            constexpr int w = decltype(W)::value;
            const uint32_t word = r.q[2 * p + w / 4][w % 4];
            const uint32_t v = word >> 8;
            const u32x2 blo = {and_or(word, 0x000F000Fu, k.k6400), and_or(v, 0x000F000Fu, k.k6400)};
            const u32x2 bhi = {and_or(word, 0x00F000F0u, k.k5400), and_or(v, 0x00F000F0u, k.k5400)};
#pragma unroll
            for (int g = 0; g < NG; g++) {
                dlo[g] = mfma_f16<w>(st.xa[p][g], blo, dlo[g]);
                dhi[g] = mfma_f16<w + 8>(st.xa[p][g], bhi, dhi[g]);
            }
        });
#pragma unroll
        for (int g = 0; g < NG; g++) {
            fma4(t[g], sc[2 * p], dlo[g]);
            fma4(t[g], sc[2 * p + 1], dhi[g]);
        }
    }
#pragma unroll
    for (int g = 0; g < NG; g++) acc[g] += t[g];
}

// One Q8_0 tile (64 rows x 128 K = four 32-element blocks).  Codes go in as 1024 + (q + 128);
// the 1152 offset comes back out through the activation sums on the fp32 matrix pipe.
template <int NG>
__device__ __forceinline__ void compute(const Stage<Q80, NG>& st, const Consts& k, float4v (&acc)[NG]) {
    const Q80::Regs& r = st.w;
    float dj[4] = {h2f_lo(r.s.x), h2f_hi(r.s.x), h2f_lo(r.s.y), h2f_hi(r.s.y)};
    float4v t[NG];
#pragma unroll
    for (int g = 0; g < NG; g++) t[g] = float4v{0.f, 0.f, 0.f, 0.f};
    static_for<4>([&](auto J) {
        constexpr int j = decltype(J)::value;
#pragma unroll
        for (int g = 0; g < NG; g++) t[g] = mfma_f32<j>(st.xs[g], dj[j] * -1152.0f, t[g]);
    });
#pragma unroll
    for (int p = 0; p < 2; p++) {
        float4v da[NG], db[NG];
#pragma unroll
        for (int g = 0; g < NG; g++) da[g] = db[g] = float4v{0.f, 0.f, 0.f, 0.f};
        static_for<8>([&](auto W) {
            constexpr int w = decltype(W)::value;
            // bytes -> fp16 1024 + (q + 128): interleave each byte with 0x64
            const uint32_t wa = r.q[4 * p + w / 4][w % 4] ^ 0x80808080u;
            const uint32_t wb = r.q[4 * p + 2 + w / 4][w % 4] ^ 0x80808080u;
            const u32x2 ba = {__builtin_amdgcn_perm(k.k64, wa, 0x04020400u), __builtin_amdgcn_perm(k.k64, wa, 0x04030401u)};
            const u32x2 bb = {__builtin_amdgcn_perm(k.k64, wb, 0x04020400u), __builtin_amdgcn_perm(k.k64, wb, 0x04030401u)};
#pragma unroll
            for (int g = 0; g < NG; g++) {
                da[g] = mfma_f16<w>(st.xa[p][g], ba, da[g]);
                db[g] = mfma_f16<w + 8>(st.xa[p][g], bb, db[g]);
            }
        });
#pragma unroll
        for (int g = 0; g < NG; g++) {
            fma4(t[g], dj[2 * p], da[g]);
            fma4(t[g], dj[2 * p + 1], db[g]);
        }
    }
#pragma unroll
    for (int g = 0; g < NG; g++) acc[g] += t[g];
}

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + __expf(-x)); }

// Stores one row group's finished sums.  v[i] is output column n of activation row 4g+i.
template <int EPI>
__device__ __forceinline__ void epilogue(const GemmArgs& a, int tile, int split, int g, float4v v, int lane, int M) {
    if (EPI == EPI_SILU) {
        // Lanes 0..31 hold the gate rows and lanes 32..63 the up rows of the same 32 columns;
        // silu(gate) * up becomes the next matmul's fp16 activation, stored in fragment order
        // together with the sum of the 32 rounded values (one whole sub-block of that matmul).
        const int col = tile * 32 + (lane & 31);  // K index of the down projection
        _Float16* out = (_Float16*)a.out;
        float* sums = (float*)((char*)a.out + xfrag_sum_offset(a.n_valid));
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float other = __shfl_xor(v[i], 32);
            const float gate = lane < 32 ? v[i] : other, up = lane < 32 ? other : v[i];
            const _Float16 h = (_Float16)(silu_f(gate) * up);
            float sum = (float)h;
#pragma unroll
            for (int o = 1; o < 32; o <<= 1) sum += __shfl_xor(sum, o);
            const int b = 4 * g + i;
            if (b < M && lane < 32) {
                out[frag_index(col, b)] = h;
                if (lane == 0) sums[xsum_index(col >> 5, b)] = sum;
            }
        }
        return;
    }
    const int n = tile * 64 + lane;
    if (n >= a.n_valid) return;
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int b = 4 * g + i;
        if (b >= M) continue;
        if (EPI == EPI_PARTIAL)
            ((float*)a.out)[((size_t)split * 16 + b) * a.ldo + n] = v[i];
        else
            ((_Float16*)a.out)[(size_t)b * a.ldo + n] = (_Float16)v[i];
    }
}

#ifndef TSV_GEMM_STAGES
#define TSV_GEMM_STAGES 2
#endif

template <class F, int EPI, int NG>
__global__ __launch_bounds__(512) void k_gemm(GemmArgs a) {
    extern __shared__ float4v red[];
    constexpr int STAGES = NG <= 2 ? TSV_GEMM_STAGES : 2;  // what fits 256 VGPRs at two waves per SIMD
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int split = blockIdx.x % a.splits, tile = blockIdx.x / a.splits;
    // this wave's run of chunks inside the workgroup's K slice
    const int s0 = split * a.kslice, s1 = min(s0 + a.kslice, a.kchunks);
    const int c0 = min(s0 + wave * a.per, s1);
    const int nc = min(a.per, s1 - c0);
    const uint8_t* wt = a.w + (size_t)tile * a.kchunks * F::TILE_BYTES;
    Consts k;
    k.k6400 = 0x64006400u;
    k.k5400 = 0x54005400u;
    k.k64 = 0x64646464u;
    asm volatile("" : "+v"(k.k6400), "+v"(k.k5400), "+v"(k.k64));

    float4v acc[NG];
#pragma unroll
    for (int g = 0; g < NG; g++) acc[g] = float4v{0.f, 0.f, 0.f, 0.f};

    // Software pipeline over the K chunks, STAGES tiles in flight per wave.  Every load in the
    // steady state is unconditional (straight-line code), so the compiler can wait on the oldest
    // outstanding tile only (s_waitcnt vmcnt(n)) instead of draining the queue.
    if (nc > 0) {
        Stage<F, NG> st[STAGES];
        const int last = c0 + nc - 1;
#pragma unroll
        for (int s = 0; s < STAGES; s++) load_stage(st[s], a, wt, min(c0 + s, last), lane);
        int c = 0;
        for (; c + 2 * STAGES <= nc; c += STAGES) {
#pragma unroll
            for (int s = 0; s < STAGES; s++) {
                compute(st[s], k, acc);
                load_stage(st[s], a, wt, c0 + c + s + STAGES, lane);
            }
        }
        // last group that still has tiles to fetch (fewer than STAGES of them)
#pragma unroll
        for (int s = 0; s < STAGES; s++) {
            if (c + s < nc) {
                compute(st[s], k, acc);
                if (c + s + STAGES < nc) load_stage(st[s], a, wt, c0 + c + s + STAGES, lane);
            }
        }
        c += STAGES;
#pragma unroll
        for (int s = 0; s < STAGES; s++)
            if (c + s < nc) compute(st[s], k, acc);
    }

    const int M = a.vp->m;
    if (a.kparts == 1) {
#pragma unroll
        for (int g = 0; g < NG; g++) epilogue<EPI>(a, tile, split, g, acc[g], lane, M);
        return;
    }
    // fold the waves' accumulators in wave order; wave w finishes row groups w, w + kparts, ...
#pragma unroll
    for (int g = 0; g < NG; g++) red[(wave * NG + g) * 64 + lane] = acc[g];
    __syncthreads();
    for (int g = wave; g < NG; g += a.kparts) {
        float4v v = red[g * 64 + lane];
        for (int w = 1; w < a.kparts; w++) v += red[(w * NG + g) * 64 + lane];
        epilogue<EPI>(a, tile, split, g, v, lane, M);
    }
}

// Chunks one wave should walk at least, by the amount of work there is to spread.
static int pref_chunks_per_wave(const TiledW& w) {
    const long total = (long)w.n_tiles * w.kchunks;
    return total >= 4096 ? 4 : total >= 2048 ? 2 : 1;
}

int gemm_default_splits(const TiledW& w, int) {
    // Independent of the row count on purpose (see the header comment).
    const int cpw = pref_chunks_per_wave(w);
    const int waves = (w.kchunks + cpw - 1) / cpw;
    int splits = std::min(8, (waves + 3) / 4);
    const int kslice = (w.kchunks + splits - 1) / splits;
    return (w.kchunks + kslice - 1) / kslice;  // every split non-empty
}

template <class F, int EPI, int NG>
static int launch_t(hipStream_t s, const GemmArgs& a) {
    const size_t lds = a.kparts > 1 ? (size_t)a.kparts * NG * 1024 : 0;
    hipLaunchKernelGGL((k_gemm<F, EPI, NG>), dim3(a.n_tiles * a.splits), dim3(64 * a.kparts), lds, s, a);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

template <class F, int EPI>
static int launch_e(hipStream_t s, const GemmArgs& a, int m) {
    if (m <= 4) return launch_t<F, EPI, 1>(s, a);
    if (m <= 8) return launch_t<F, EPI, 2>(s, a);
    return launch_t<F, EPI, 4>(s, a);
}

template <class F>
static int launch_f(hipStream_t s, const GemmArgs& a, int m, int epi) {
    switch (epi) {
        case EPI_PARTIAL: return launch_e<F, EPI_PARTIAL>(s, a, m);
        case EPI_SILU: return launch_e<F, EPI_SILU>(s, a, m);
        default: return launch_e<F, EPI_LOGITS>(s, a, m);
    }
}

int launch_gemm(hipStream_t s, const TiledW& w, const uint4* xfrag, void* out, const VerifyParams* vp,
                int m, int splits, int epi, int ldo, int n_valid) {
    if (m < 1 || m > TSV_MAX_ROWS) {
        set_error("matmul: row count outside 1..16");
        return TSV_ERR_INVALID;
    }
    if (epi != EPI_PARTIAL) splits = 1;
    if (splits < 1) splits = 1;
    if (splits > w.kchunks) splits = w.kchunks;
    GemmArgs a;
    a.w = w.tiles;
    a.xfrag = (const uint2*)xfrag;
    a.xsum = (const float*)((const char*)xfrag + xfrag_sum_offset(w.k));
    a.out = out;
    a.vp = vp;
    a.n_tiles = w.n_tiles;
    a.kchunks = w.kchunks;
    a.kslice = (w.kchunks + splits - 1) / splits;
    a.splits = (w.kchunks + a.kslice - 1) / a.kslice;
    if (epi == EPI_PARTIAL && a.splits != splits) {
        set_error("matmul: split count leaves an empty K slice");
        return TSV_ERR_INVALID;
    }
    const int cpw = pref_chunks_per_wave(w);
    int kparts = std::min(8, std::max(1, (a.kslice + cpw - 1) / cpw));
    a.per = (a.kslice + kparts - 1) / kparts;
    a.kparts = (a.kslice + a.per - 1) / a.per;
    a.ldo = ldo;
    a.n_valid = n_valid;
    if (epi == EPI_SILU) {
        if (w.n_rows % 64) {
            set_error("matmul: gate/up rows must fill whole 64-row tiles");
            return TSV_ERR_INVALID;
        }
        a.n_valid = w.n_rows / 2;  // K of the next matmul
    }
    return w.fmt == FMT_Q4K ? launch_f<Q4K>(s, a, m, epi) : launch_f<Q80>(s, a, m, epi);
}

}  // namespace tsv
