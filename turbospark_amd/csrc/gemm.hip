// Dequant-fused small-M matmul for GGUF Q4_K / Q8_0 weights on gfx950 (wave64, MFMA).
//
// Replaces the reference's batched verify GEMM (crates/gpu/src/shaders/dequant_kquant_batch.metal:62-123,
// host wrapper dequant_kquant_gemm_batch.rs:96-126): Y[b][n] = sum_k W[n][k] * X[b][k], b < 16,
// every weight byte read once for all rows.  The arithmetic contract is the CPU reference's
// (crates/compute/src/quant_gguf/q4_k.rs:67-108,207-220; q8_0.rs:19-47,80-93).
//
// How it maps to the hardware:
//  * one wave owns a 16-row tile and walks K; per 32-element sub-block it issues ONE
//    v_mfma_f32_16x16x32_f16 with the (<=16) activation rows as the A operand and the 16 weight
//    rows as the B operand, so the MAC work rides the matrix pipe and the vector ALUs only
//    unpack nibbles and apply block scales;
//  * quant codes go to the MFMA as exact fp16 integers: (v & 0x000F000F) | 0x64006400 is the
//    pair (1024+q, 1024+q'), (v & 0x00F000F0) | 0x54005400 is (64+q, 64+q') -- one
//    v_and_or_b32 per two weights, no int->float convert; the offset is removed in fp32 through
//    the per-sub-block activation sums that the Q4_K min term needs anyway:
//        y += d*sc_j * D_j - (d*sc_j*off + dmin*m_j) * sum_k x_k
//  * the element order inside an 8-wide K slice is whatever the unpack produces
//    ([0,2,1,3,4,6,5,7]); the activations are stored pre-permuted instead of shuffling weights;
//  * weights are re-tiled once at load so each wave-wide load is 1 KiB contiguous (16 B per
//    lane); activations for the workgroup's K slice are staged once in LDS and shared by its waves.
#include <algorithm>

#include "tsv_internal.h"

namespace tsv {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

// ------------------------------------------------------------------------------- re-tiling
// One thread per 16-byte unit of the output tile.
__global__ void k_repack_q4k(const uint8_t* __restrict__ raw, int n_rows, int kchunks,
                             uint8_t* __restrict__ tiles, int tile_stride, int tile_offset,
                             int n_src_tiles) {
    long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    long total = (long)n_src_tiles * kchunks * 144;
    if (gid >= total) return;
    int c = (int)(gid % 144);
    long t = gid / 144;
    int sb = (int)(t % kchunks);
    int st = (int)(t / kchunks);
    uint8_t* dst = tiles + (((long)(st * tile_stride + tile_offset)) * kchunks + sb) * 2304 + (long)c * 16;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (c < 128) {
        int h = c >> 6, lane = c & 63, r = lane & 15, kg = lane >> 4;
        int row = st * 16 + r;
        if (row < n_rows) {
            const uint8_t* blk = raw + ((long)row * kchunks + sb) * 144 + 16;
            const uint2 a = *(const uint2*)(blk + 32 * (2 * h) + 8 * kg);
            const uint2 b = *(const uint2*)(blk + 32 * (2 * h + 1) + 8 * kg);
            v = make_uint4(a.x, a.y, b.x, b.y);
        }
    } else {
        int r = c - 128;
        int row = st * 16 + r;
        if (row < n_rows) v = *(const uint4*)(raw + ((long)row * kchunks + sb) * 144);
    }
    *(uint4*)dst = v;
}

__global__ void k_repack_q80(const uint8_t* __restrict__ raw, int n_rows, int kchunks,
                             uint8_t* __restrict__ tiles, int tile_stride, int tile_offset,
                             int n_src_tiles) {
    long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    long total = (long)n_src_tiles * kchunks * 136;
    if (gid >= total) return;
    int c = (int)(gid % 136);
    long t = gid / 136;
    int kt = (int)(t % kchunks);
    int st = (int)(t / kchunks);
    uint8_t* dst = tiles + (((long)(st * tile_stride + tile_offset)) * kchunks + kt) * 2176 + (long)c * 16;
    long row_bytes = (long)kchunks * 4 * 34;
    if (c < 128) {
        int h = c >> 6, lane = c & 63, r = lane & 15, kg = lane >> 4;
        int row = st * 16 + r;
        uint8_t tmp[16];
#pragma unroll
        for (int i = 0; i < 16; i++) tmp[i] = 0;
        if (row < n_rows) {
            const uint8_t* b0 = raw + row * row_bytes + (long)(kt * 4 + 2 * h) * 34 + 2 + 8 * kg;
            const uint8_t* b1 = b0 + 34;
#pragma unroll
            for (int i = 0; i < 8; i++) {
                tmp[i] = b0[i];
                tmp[8 + i] = b1[i];
            }
        }
#pragma unroll
        for (int i = 0; i < 16; i++) dst[i] = tmp[i];
    } else {
        int cc = c - 128;  // rows 2cc, 2cc+1
#pragma unroll
        for (int rr = 0; rr < 2; rr++) {
            int row = st * 16 + 2 * cc + rr;
#pragma unroll
            for (int b = 0; b < 4; b++) {
                uint16_t d = 0;
                if (row < n_rows) {
                    const uint8_t* p = raw + row * row_bytes + (long)(kt * 4 + b) * 34;
                    d = (uint16_t)(p[0] | (p[1] << 8));
                }
                *(uint16_t*)(dst + rr * 8 + b * 2) = d;
            }
        }
    }
}

int launch_repack(hipStream_t s, int fmt, const uint8_t* raw, int n_rows, int k, uint8_t* tiles,
                  int kchunks, int tile_stride, int tile_offset) {
    int n_src_tiles = (n_rows + 15) / 16;
    if (fmt == FMT_Q4K) {
        long total = (long)n_src_tiles * kchunks * 144;
        hipLaunchKernelGGL(k_repack_q4k, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, raw,
                           n_rows, kchunks, tiles, tile_stride, tile_offset, n_src_tiles);
    } else {
        long total = (long)n_src_tiles * kchunks * 136;
        hipLaunchKernelGGL(k_repack_q80, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, raw,
                           n_rows, kchunks, tiles, tile_stride, tile_offset, n_src_tiles);
    }
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

// ------------------------------------------------------------------------------- formats
struct Q4K {
    static constexpr int NSUB = 8, TILE_BYTES = 2304;
    struct Regs {
        u32x4 q0, q1, s;
    };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* tile, int lane) {
        const u32x4* p = (const u32x4*)tile;
        r.q0 = __builtin_nontemporal_load(p + lane);
        r.q1 = __builtin_nontemporal_load(p + 64 + lane);
        r.s = __builtin_nontemporal_load(p + 128 + (lane & 15));
    }
};

struct Q80 {
    static constexpr int NSUB = 4, TILE_BYTES = 2176;
    struct Regs {
        u32x4 q0, q1;
        u32x2 s;
    };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* tile, int lane) {
        const u32x4* p = (const u32x4*)tile;
        r.q0 = __builtin_nontemporal_load(p + lane);
        r.q1 = __builtin_nontemporal_load(p + 64 + lane);
        r.s = __builtin_nontemporal_load((const u32x2*)(tile + 2048) + (lane & 15));
    }
};

__device__ __forceinline__ float h2f_lo(uint32_t v) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(v & 0xFFFF));
}
__device__ __forceinline__ float h2f_hi(uint32_t v) {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)(v >> 16));
}
__device__ __forceinline__ float ubyte(uint32_t v, int i) { return (float)((v >> (8 * i)) & 0xFF); }

__device__ __forceinline__ half8 as_half8(uint4 v) { return __builtin_bit_cast(half8, v); }
__device__ __forceinline__ half8 as_half8(u32x4 v) { return __builtin_bit_cast(half8, v); }

// (v & mask) | bits as ONE v_and_or_b32: the instruction can take a single literal / scalar
// operand, so the second constant is pinned in a vector register.
__device__ __forceinline__ uint32_t and_or(uint32_t v, uint32_t mask, uint32_t bits_vgpr) {
    return (v & mask) | bits_vgpr;
}

struct Consts {
    uint32_t k6400, k5400, k64;
};

// One Q4_K superblock tile (16 weight rows x 256 K) against the staged activations.
//   acc  += sum_j d*sc_j * (X_j . (off_j + q_j))          8 x v_mfma_f32_16x16x32_f16 + 4 FMAs each
//   acc  -= sum_j (d*sc_j*off_j + dmin*m_j) * sum_k X_jk   2 x v_mfma_f32_16x16x4_f32 (fp32 operands,
//           K index = sub-block: lane group kg supplies sub-blocks kg and 4+kg)
// Both parts are summed per tile first so the large code offsets cancel before they reach the
// running accumulator.
__device__ __forceinline__ void compute(const Q4K::Regs& r, const uint4* xf, const float* xs, int lc, int lane,
                                        int M, int rowA, const Consts& k, float4v& acc) {
    const int kg = lane >> 4;
    float4v t;  // this tile's contribution: starts at the (negative) offset term, ends small
    const float d = h2f_lo(r.s.x), dmin = h2f_hi(r.s.x);
    // 6-bit scale / min unpack (q4_k.rs:43-54), four sub-blocks per 32-bit word
    const uint32_t sl = r.s.y & 0x3F3F3F3Fu, ml = r.s.z & 0x3F3F3F3Fu;
    const uint32_t sh = (r.s.w & 0x0F0F0F0Fu) | ((r.s.y >> 2) & 0x30303030u);
    const uint32_t mh = ((r.s.w >> 4) & 0x0F0F0F0Fu) | ((r.s.z >> 2) & 0x30303030u);
    const float4v zero = {0.f, 0.f, 0.f, 0.f};
    // min / offset term: this lane's two sub-blocks are kg (from sl/ml) and 4+kg (from sh/mh);
    // even sub-blocks carry the 1024 code offset, odd ones 64.
    {
        const float off = (kg & 1) ? 64.0f : 1024.0f;
        const float s0 = d * (float)((sl >> (8 * kg)) & 0xFFu), s1 = d * (float)((sh >> (8 * kg)) & 0xFFu);
        const float c0 = __builtin_fmaf(s0, off, dmin * (float)((ml >> (8 * kg)) & 0xFFu));
        const float c1 = __builtin_fmaf(s1, off, dmin * (float)((mh >> (8 * kg)) & 0xFFu));
        const float x0 = xs[(lc * 8 + kg) * M + rowA], x1 = xs[(lc * 8 + 4 + kg) * M + rowA];
        t = __builtin_amdgcn_mfma_f32_16x16x4f32(x0, -c0, zero, 0, 0, 0);
        t = __builtin_amdgcn_mfma_f32_16x16x4f32(x1, -c1, t, 0, 0, 0);
    }
#pragma unroll
    for (int g = 0; g < 4; g++) {
        const uint32_t w0 = g == 0 ? r.q0.x : g == 1 ? r.q0.z : g == 2 ? r.q1.x : r.q1.z;
        const uint32_t w1 = g == 0 ? r.q0.y : g == 1 ? r.q0.w : g == 2 ? r.q1.y : r.q1.w;
        const uint32_t sw = g < 2 ? sl : sh;
        const int b0 = (2 * g) & 3;
        const uint32_t v0 = w0 >> 8, v1 = w1 >> 8;
        // low nibbles: sub-block 2g, codes as 1024+q
        {
            uint4 b = make_uint4(and_or(w0, 0x000F000Fu, k.k6400), and_or(v0, 0x000F000Fu, k.k6400),
                                 and_or(w1, 0x000F000Fu, k.k6400), and_or(v1, 0x000F000Fu, k.k6400));
            const uint4 a = xf[((lc * 8 + 2 * g) * 4 + kg) * M + rowA];
            const float4v D = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(a), as_half8(b), zero, 0, 0, 0);
            const float sj = d * ubyte(sw, b0);
            t.x = __builtin_fmaf(sj, D.x, t.x);
            t.y = __builtin_fmaf(sj, D.y, t.y);
            t.z = __builtin_fmaf(sj, D.z, t.z);
            t.w = __builtin_fmaf(sj, D.w, t.w);
        }
        // high nibbles: sub-block 2g+1, codes as 64+q
        {
            uint4 b = make_uint4(and_or(w0, 0x00F000F0u, k.k5400), and_or(v0, 0x00F000F0u, k.k5400),
                                 and_or(w1, 0x00F000F0u, k.k5400), and_or(v1, 0x00F000F0u, k.k5400));
            const uint4 a = xf[((lc * 8 + 2 * g + 1) * 4 + kg) * M + rowA];
            const float4v D = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(a), as_half8(b), zero, 0, 0, 0);
            const float sj = d * ubyte(sw, b0 + 1);
            t.x = __builtin_fmaf(sj, D.x, t.x);
            t.y = __builtin_fmaf(sj, D.y, t.y);
            t.z = __builtin_fmaf(sj, D.z, t.z);
            t.w = __builtin_fmaf(sj, D.w, t.w);
        }
    }
    acc += t;
}

// One Q8_0 tile (16 rows x 128 K = four 32-element blocks).  Codes go in as 1024 + (q + 128);
// the 1152 offset comes back out through the activation sums on the fp32 matrix pipe.
__device__ __forceinline__ void compute(const Q80::Regs& r, const uint4* xf, const float* xs, int lc, int lane,
                                        int M, int rowA, const Consts& k, float4v& acc) {
    const int kg = lane >> 4;
    float4v t;
    const float4v zero = {0.f, 0.f, 0.f, 0.f};
    {
        const uint32_t sw = kg < 2 ? r.s.x : r.s.y;
        const float dk = (kg & 1) ? h2f_hi(sw) : h2f_lo(sw);  // block kg's scale
        t = __builtin_amdgcn_mfma_f32_16x16x4f32(xs[(lc * 4 + kg) * M + rowA], dk * -1152.0f, zero, 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t w0 = (j == 0 ? r.q0.x : j == 1 ? r.q0.z : j == 2 ? r.q1.x : r.q1.z) ^ 0x80808080u;
        const uint32_t w1 = (j == 0 ? r.q0.y : j == 1 ? r.q0.w : j == 2 ? r.q1.y : r.q1.w) ^ 0x80808080u;
        // bytes -> fp16 1024 + (q + 128): interleave each byte with 0x64
        uint4 b = make_uint4(__builtin_amdgcn_perm(k.k64, w0, 0x04020400u), __builtin_amdgcn_perm(k.k64, w0, 0x04030401u),
                             __builtin_amdgcn_perm(k.k64, w1, 0x04020400u), __builtin_amdgcn_perm(k.k64, w1, 0x04030401u));
        const uint4 a = xf[((lc * 4 + j) * 4 + kg) * M + rowA];
        const float4v D = __builtin_amdgcn_mfma_f32_16x16x32_f16(as_half8(a), as_half8(b), zero, 0, 0, 0);
        const uint32_t sw = j < 2 ? r.s.x : r.s.y;
        const float dj = (j & 1) ? h2f_hi(sw) : h2f_lo(sw);
        t.x = __builtin_fmaf(dj, D.x, t.x);
        t.y = __builtin_fmaf(dj, D.y, t.y);
        t.z = __builtin_fmaf(dj, D.z, t.z);
        t.w = __builtin_fmaf(dj, D.w, t.w);
    }
    acc += t;
}

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + __expf(-x)); }

// Position of K element `e` (0..31 inside a sub-block) in the fragment buffer, in halfs,
// relative to the sub-block's base: [kg][16 rows][8] with the unpack permutation.
__device__ __forceinline__ int frag_off(int e, int row) {
    const int kg = e >> 3, o = e & 7;
    const int p = (o & 4) | ((o & 1) << 1) | ((o >> 1) & 1);  // [0,2,1,3,4,6,5,7], an involution
    return (kg * 16 + row) * 8 + p;
}

// LDS bytes per 32-element sub-block of a K slice for m activation rows: fp16 fragments + fp32 sums.
__host__ __device__ inline int lds_per_sub(int m) { return 4 * m * 16 + m * 4; }

#ifndef TSV_GEMM_STAGES
#define TSV_GEMM_STAGES 4
#endif
#ifndef TSV_GEMM_WAVES
#define TSV_GEMM_WAVES 2
#endif

template <class F, int EPI>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(TSV_GEMM_WAVES, TSV_GEMM_WAVES)))
void k_gemm(GemmArgs a) {
    extern __shared__ uint4 lds[];
    constexpr int STAGES = TSV_GEMM_STAGES;
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int split = blockIdx.x % a.splits, grp = blockIdx.x / a.splits;
    const int tile = grp * 4 + wave;
    const int c0 = split * a.kslice;
    const int nc = min(a.kslice, a.kchunks - c0);
    const bool active = tile < a.n_tiles && nc > 0;
    const uint8_t* wt = a.w + ((size_t)tile * a.kchunks + c0) * F::TILE_BYTES;
    const int M = a.vp->m;
    const int rowA = min(lane & 15, M - 1);  // padding rows of the A operand alias the last real row
    Consts k;
    k.k6400 = 0x64006400u;
    k.k5400 = 0x54005400u;
    k.k64 = 0x64646464u;
    asm volatile("" : "+v"(k.k6400), "+v"(k.k5400), "+v"(k.k64));

    // Software pipeline over the K chunks, STAGES tiles in flight per wave.  Every load in the
    // steady state is unconditional (straight-line code), so the compiler can wait on the oldest
    // outstanding tile only (s_waitcnt vmcnt(n)) instead of draining the queue.
    typename F::Regs st[STAGES];
    const int last = max(nc - 1, 0);
    if (active) {
#pragma unroll
        for (int s = 0; s < STAGES; s++) F::load(st[s], wt + (size_t)min(s, last) * F::TILE_BYTES, lane);
    }

    // stage this K slice of the activations: [sub][kg][M rows] x 16 B, then their per-sub-block sums
    const int nsub = nc * F::NSUB, sub0 = c0 * F::NSUB;
    uint4* xf = lds;
    float* xs = (float*)(lds + a.kslice * F::NSUB * 4 * M);
    for (int u = tid; u < nsub * 4 * M; u += 256) {
        const int row = u % M, t = u / M;
        xf[u] = a.xfrag[((size_t)(sub0 * 4 + t)) * 16 + row];
    }
    __syncthreads();
    for (int v = tid; v < nsub * M; v += 256) {
        const int row = v % M, ls = v / M;
        float s = 0.f;
#pragma unroll
        for (int kg = 0; kg < 4; kg++) {
            const half8 h = as_half8(xf[(ls * 4 + kg) * M + row]);
#pragma unroll
            for (int i = 0; i < 8; i++) s += (float)h[i];
        }
        xs[v] = s;
    }
    __syncthreads();

    float4v acc = {0.f, 0.f, 0.f, 0.f};
    if (active) {
        int c = 0;
        for (; c + 2 * STAGES <= nc; c += STAGES) {
#pragma unroll
            for (int s = 0; s < STAGES; s++) {
                compute(st[s], xf, xs, c + s, lane, M, rowA, k, acc);
                F::load(st[s], wt + (size_t)(c + s + STAGES) * F::TILE_BYTES, lane);
            }
        }
        // last group that still has tiles to fetch (fewer than STAGES of them)
#pragma unroll
        for (int s = 0; s < STAGES; s++) {
            if (c + s < nc) {
                compute(st[s], xf, xs, c + s, lane, M, rowA, k, acc);
                if (c + s + STAGES < nc) F::load(st[s], wt + (size_t)(c + s + STAGES) * F::TILE_BYTES, lane);
            }
        }
        c += STAGES;
#pragma unroll
        for (int s = 0; s < STAGES; s++)
            if (c + s < nc) compute(st[s], xf, xs, c + s, lane, M, rowA, k, acc);
    }

    const int j = lane & 15, kg = lane >> 4;
    const int n = tile * 16 + j;
    const int m = M;
    if (EPI == EPI_PARTIAL) {
        if (!active) return;
        float* out = (float*)a.out + (size_t)split * 16 * a.ldo;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int b = 4 * kg + i;
            if (b < m) out[(size_t)b * a.ldo + n] = acc[i];
        }
    } else if (EPI == EPI_LOGITS) {
        if (!active || n >= a.n_valid) return;
        _Float16* out = (_Float16*)a.out;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int b = 4 * kg + i;
            if (b < m) out[(size_t)b * a.ldo + n] = (_Float16)acc[i];
        }
    } else {
        // gate / up row tiles alternate (even = gate, odd = up): the odd wave hands its
        // accumulators to the even one through LDS, which stores silu(gate) * up as the next
        // matmul's fp16 activation fragments.
        __syncthreads();
        float4v* ex = (float4v*)lds;
        if (wave & 1) ex[(wave >> 1) * 64 + lane] = acc;
        __syncthreads();
        if (!(wave & 1) && active) {
            const float4v up = ex[(wave >> 1) * 64 + lane];
            const int col = (tile >> 1) * 16 + j;  // K index of the down projection
            _Float16* out = (_Float16*)a.out + (size_t)(col >> 5) * (4 * 16 * 8);
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int b = 4 * kg + i;
                if (b < m) out[frag_off(col & 31, b)] = (_Float16)(silu_f(acc[i]) * up[i]);
            }
        }
    }
}

int gemm_default_splits(const TiledW& w, int m) {
    // Enough workgroups to cover 256 CUs about twice, K slices no shorter than two chunks,
    // and an LDS footprint that still lets several workgroups share a CU.
    const int groups = (w.n_tiles + 3) / 4;
    int splits = 1;
    while (groups * splits < 448 && w.kchunks / (splits * 2) >= 2 && w.kchunks % (splits * 2) == 0) splits *= 2;
    // odd chunk counts (e.g. 56 = 7 * 8): allow a non power of two that divides evenly
    if (groups * splits < 448)
        for (int s = splits + 1; s <= w.kchunks / 2; s++)
            if (w.kchunks % s == 0 && groups * s <= 640) {
                splits = s;
                if (groups * s >= 448) break;
            }
    const int chunk_bytes = fmt_nsub(w.fmt) * lds_per_sub(m);
    while ((w.kchunks + splits - 1) / splits * chunk_bytes > 76 * 1024) splits++;
    // normalise: every split non-empty
    const int kslice = (w.kchunks + splits - 1) / splits;
    return (w.kchunks + kslice - 1) / kslice;
}

template <class F, int EPI>
static int launch_t(hipStream_t s, const GemmArgs& a, int groups, int m) {
    const size_t lds = std::max<size_t>((size_t)a.kslice * F::NSUB * lds_per_sub(m), 2048);
    static bool configured = false;
    if (!configured) {
        TSV_HIP(hipFuncSetAttribute((const void*)k_gemm<F, EPI>, hipFuncAttributeMaxDynamicSharedMemorySize,
                                    (int)(160 * 1024)));
        configured = true;
    }
    if (lds > 160 * 1024) {
        set_error("matmul: activation slice does not fit LDS; raise the split count");
        return TSV_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL((k_gemm<F, EPI>), dim3(groups * a.splits), dim3(256), lds, s, a);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

template <class F>
static int launch_f(hipStream_t s, const GemmArgs& a, int groups, int m, int epi) {
    switch (epi) {
        case EPI_PARTIAL: return launch_t<F, EPI_PARTIAL>(s, a, groups, m);
        case EPI_SILU: return launch_t<F, EPI_SILU>(s, a, groups, m);
        default: return launch_t<F, EPI_LOGITS>(s, a, groups, m);
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
    a.xfrag = xfrag;
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
    a.ldo = ldo;
    a.n_valid = n_valid;
    const int groups = (w.n_tiles + 3) / 4;
    return w.fmt == FMT_Q4K ? launch_f<Q4K>(s, a, groups, m, epi) : launch_f<Q80>(s, a, groups, m, epi);
}

}  // namespace tsv
