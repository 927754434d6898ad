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
#include <cstdlib>

#include "gemm_core.h"

namespace tsv {

// ------------------------------------------------------------------------------- re-tiling
// One thread per 16-byte unit of a source row's chunk (unit 8 = the scale header).
__global__ void k_repack_q4k(const uint8_t* __restrict__ raw, int n_rows, int kchunks,
                             uint8_t* __restrict__ tiles, int grp, int stride, int offset, const int32_t* __restrict__ rowmap) {
    const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long total = (long)n_rows * kchunks * 9;
    if (gid >= total) return;
    const int u = (int)(gid % 9);
    const long t = gid / 9;
    const int c = (int)(t % kchunks);
    const int r = (int)(t / kchunks);
    const int drow = rowmap ? rowmap[r] : (r / grp) * stride + offset + r % grp;
    const int tile = drow >> 6, lane = drow & 63;
    const uint8_t* blk = raw + ((long)r * kchunks + c) * 144;
    uint8_t* dst = tiles + ((long)tile * kchunks + c) * 9216 + (u < 8 ? (u * 64 + lane) * 16 : 8192 + lane * 16);
    *(uint4*)dst = *(const uint4*)(u < 8 ? blk + 16 + 16 * u : blk);
}

// Q5_K: units 0..7 the nibble bytes, 8 the scale header (both as in Q4_K), 9 and 10 the fifth bits.
__global__ void k_repack_q5k(const uint8_t* __restrict__ raw, int n_rows, int kchunks,
                             uint8_t* __restrict__ tiles, int grp, int stride, int offset, const int32_t* __restrict__ rowmap) {
    const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long total = (long)n_rows * kchunks * 11;
    if (gid >= total) return;
    const int u = (int)(gid % 11);
    const long t = gid / 11;
    const int c = (int)(t % kchunks);
    const int r = (int)(t / kchunks);
    const int drow = rowmap ? rowmap[r] : (r / grp) * stride + offset + r % grp;
    const int tile = drow >> 6, lane = drow & 63;
    const uint8_t* blk = raw + ((long)r * kchunks + c) * 176;
    uint8_t* dst = tiles + ((long)tile * kchunks + c) * 11264 + (u * 64 + lane) * 16;
    *(uint4*)dst = *(const uint4*)(u < 8 ? blk + 48 + 16 * u : u == 8 ? blk : blk + 16 + 16 * (u - 9));
}

__global__ void k_repack_q80(const uint8_t* __restrict__ raw, int n_rows, int kchunks,
                             uint8_t* __restrict__ tiles, int grp, int stride, int offset, const int32_t* __restrict__ rowmap) {
    const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long total = (long)n_rows * kchunks * 9;
    if (gid >= total) return;
    const int u = (int)(gid % 9);
    const long t = gid / 9;
    const int c = (int)(t % kchunks);
    const int r = (int)(t / kchunks);
    const int drow = rowmap ? rowmap[r] : (r / grp) * stride + offset + r % grp;
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

// MXFP4: one thread per source block (17 bytes: scale, then 16 bytes whose low / high nibbles are
// elements j and j + 16).  Nibble n of output word w is K element 8w + {0,2,1,3,4,6,5,7}[n].
__global__ void k_repack_mx4(const uint8_t* __restrict__ raw, int n_rows, int kchunks,
                             uint8_t* __restrict__ tiles, int grp, int stride, int offset, int nblk,
                             const int32_t* __restrict__ rowmap) {
    const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long total = (long)n_rows * kchunks * 8;
    if (gid >= total) return;
    const int u = (int)(gid % 8);
    const long t = gid / 8;
    const int c = (int)(t % kchunks);
    const int r = (int)(t / kchunks);
    const int drow = rowmap ? rowmap[r] : (r / grp) * stride + offset + r % grp;
    const int tile = drow >> 6, lane = drow & 63;
    if (c * 8 + u >= nblk) return;  // past the row's last block: the tile keeps its zero block
    const uint8_t* blk = raw + ((long)r * nblk + (long)c * 8 + u) * 17;
    uint8_t* tb = tiles + ((long)tile * kchunks + c) * 8704;
    uint32_t words[4];
#pragma unroll
    for (int w = 0; w < 4; w++) {
        uint32_t v = 0;
#pragma unroll
        for (int n = 0; n < 8; n++) {
            const int k = 8 * w + ((n & 4) | ((n & 1) << 1) | ((n >> 1) & 1));
            const uint32_t code = k < 16 ? (blk[1 + k] & 0xFu) : (uint32_t)(blk[1 + k - 16] >> 4);
            v |= code << (4 * n);
        }
        words[w] = v;
    }
    *(uint4*)(tb + (u * 64 + lane) * 16) = make_uint4(words[0], words[1], words[2], words[3]);
    tb[8192 + lane * 8 + u] = blk[0];
}

// Q6_K: one thread per unit of a (row, chunk): 12 quant units, the scale unit, the d word.
__device__ __forceinline__ uint32_t q6k_level(const uint8_t* blk, int e) {
    // q6_k.rs:67-84: element e = 128 h + 32 k + l takes its low nibble from ql[64 h + l + 32 (k & 1)]
    // (upper nibble when k >= 2) and its high pair from bits 2k.. of qh[32 h + l]
    const int h = e >> 7, k = (e >> 5) & 3, l = e & 31;
    const uint32_t lo = (blk[64 * h + l + 32 * (k & 1)] >> (4 * (k >> 1))) & 0xFu;
    const uint32_t hi = (blk[128 + 32 * h + l] >> (2 * k)) & 3u;
    return lo | (hi << 4);
}
__global__ void k_repack_q6k(const uint8_t* __restrict__ raw, int n_rows, int kchunks,
                             uint8_t* __restrict__ tiles, int grp, int stride, int offset, const int32_t* __restrict__ rowmap) {
    const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long total = (long)n_rows * kchunks * 14;
    if (gid >= total) return;
    const int u = (int)(gid % 14);
    const long t = gid / 14;
    const int c = (int)(t % kchunks);
    const int r = (int)(t / kchunks);
    const int drow = rowmap ? rowmap[r] : (r / grp) * stride + offset + r % grp;
    const int tile = drow >> 6, lane = drow & 63;
    const uint8_t* blk = raw + ((long)r * kchunks + c) * 210;
    uint8_t* tb = tiles + ((long)tile * kchunks + c) * 13568;
    if (u == 13) {
        *(uint32_t*)(tb + 13312 + lane * 4) = (uint32_t)blk[208] | ((uint32_t)blk[209] << 8);
        return;
    }
    if (u == 12) {
        uint32_t w[4];
#pragma unroll
        for (int i = 0; i < 4; i++)
            w[i] = (uint32_t)blk[192 + 4 * i] | ((uint32_t)blk[193 + 4 * i] << 8) | ((uint32_t)blk[194 + 4 * i] << 16) |
                   ((uint32_t)blk[195 + 4 * i] << 24);
        *(uint4*)(tb + 12288 + lane * 16) = make_uint4(w[0], w[1], w[2], w[3]);
        return;
    }
    const int p = u / 3, part = u % 3;
    uint32_t w[4] = {0, 0, 0, 0};
    if (part < 2) {
        // word i: steps a = 8 part + 2i and a + 1; nibbles k0 k1 (a), k0 k1 (a + 1), k2 k3 (a), k2 k3 (a + 1)
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int e0 = 64 * p + 4 * (8 * part + 2 * i);
            const int order[8] = {e0, e0 + 1, e0 + 4, e0 + 5, e0 + 2, e0 + 3, e0 + 6, e0 + 7};
#pragma unroll
            for (int n = 0; n < 8; n++) w[i] |= (q6k_level(blk, order[n]) & 0xFu) << (4 * n);
        }
    } else {
        // word i: steps 4i .. 4i + 3; extraction e = 2 * (step % 4) + ab holds (k0, k2) for ab = 0 and
        // (k1, k3) for ab = 1: the first element's pair at bits 2e, the second's at bits 16 + 2e
#pragma unroll
        for (int i = 0; i < 4; i++)
#pragma unroll
            for (int si = 0; si < 4; si++)
#pragma unroll
                for (int ab = 0; ab < 2; ab++) {
                    const int e0 = 64 * p + 4 * (4 * i + si), e = 2 * si + ab;
                    w[i] |= (q6k_level(blk, e0 + ab) >> 4) << (2 * e);
                    w[i] |= (q6k_level(blk, e0 + 2 + ab) >> 4) << (16 + 2 * e);
                }
    }
    *(uint4*)(tb + (u * 64 + lane) * 16) = make_uint4(w[0], w[1], w[2], w[3]);
}

// bf16: one thread per 16-byte unit (eight consecutive K values of a row, two MFMA steps).
__global__ void k_repack_bf16(const uint8_t* __restrict__ raw, int n_rows, int kchunks,
                              uint8_t* __restrict__ tiles, int grp, int stride, int offset, const int32_t* __restrict__ rowmap) {
    const long gid = (long)blockIdx.x * blockDim.x + threadIdx.x;
    const long total = (long)n_rows * kchunks * 8;
    if (gid >= total) return;
    const int u = (int)(gid % 8);
    const long t = gid / 8;
    const int c = (int)(t % kchunks);
    const int r = (int)(t / kchunks);
    const int drow = rowmap ? rowmap[r] : (r / grp) * stride + offset + r % grp;
    const int tile = drow >> 6, lane = drow & 63;
    const uint16_t* src = (const uint16_t*)raw + ((long)r * kchunks + c) * 64 + 8 * u;
    uint16_t v[8];
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = src[(i & 4) | ((i & 1) << 1) | ((i >> 1) & 1)];
    uint16_t* dst = (uint16_t*)(tiles + ((long)tile * kchunks + c) * 8192 + (u * 64 + lane) * 16);
#pragma unroll
    for (int i = 0; i < 8; i++) dst[i] = v[i];
}

int launch_repack(hipStream_t s, int fmt, const uint8_t* raw, int n_rows, int k, uint8_t* tiles,
                  int kchunks, int grp, int stride, int offset, const int32_t* rowmap) {
    const long total = (long)n_rows * kchunks * 9;
    if (total == 0) return TSV_OK;
    if (fmt == FMT_Q6K) {
        const long units = (long)n_rows * kchunks * 14;
        hipLaunchKernelGGL(k_repack_q6k, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, s, raw, n_rows, kchunks,
                           tiles, grp, stride, offset, rowmap);
    } else if (fmt == FMT_BF16) {
        const long units = (long)n_rows * kchunks * 8;
        hipLaunchKernelGGL(k_repack_bf16, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, s, raw, n_rows, kchunks,
                           tiles, grp, stride, offset, rowmap);
    } else if (fmt == FMT_MX4) {
        const long blocks = (long)n_rows * kchunks * 8;
        hipLaunchKernelGGL(k_repack_mx4, dim3((unsigned)((blocks + 255) / 256)), dim3(256), 0, s, raw, n_rows, kchunks,
                           tiles, grp, stride, offset, k / 32, rowmap);
    } else if (fmt == FMT_Q5K) {
        const long units = (long)n_rows * kchunks * 11;
        hipLaunchKernelGGL(k_repack_q5k, dim3((unsigned)((units + 255) / 256)), dim3(256), 0, s, raw, n_rows, kchunks,
                           tiles, grp, stride, offset, rowmap);
    } else if (fmt == FMT_Q4K)
        hipLaunchKernelGGL(k_repack_q4k, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, raw, n_rows,
                           kchunks, tiles, grp, stride, offset, rowmap);
    else
        hipLaunchKernelGGL(k_repack_q80, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, s, raw, n_rows,
                           kchunks, tiles, grp, stride, offset, rowmap);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

// Stores one row group's finished sums.  v[i] is output column n of activation row 4g+i.
template <int EPI>
__device__ __forceinline__ void epilogue(const GemmArgs& a, int tile, int split, int g, float4v v, int lane, int M) {
    if (EPI == EPI_ROPE) {
        rope_epilogue(a.rope, a.vp, tile, g, v, lane, M);
        return;
    }
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
            const _Float16 h = pinned_half((_Float16)(silu_f(gate) * up));
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

// Tiles in flight per wave.  One: up to eight activation rows then fit 128 VGPRs, so four waves
// per SIMD are resident instead of two, and inside a verify step (cold L2 and TLB at every launch)
// that hides more latency than a second register stage does -- the 8B step went from 2.31 to
// 2.23 ms on the same box, the 16-row tree step from 3.62 to 3.51 ms (there the kernel stays at two
// waves per SIMD either way), although an isolated launch on warm caches times the same.
#ifndef TSV_GEMM_STAGES
#define TSV_GEMM_STAGES 1
#endif

template <class F, int EPI, int NG>
__global__ __launch_bounds__(512) void k_gemm(GemmArgs a) {
    extern __shared__ float4v red[];
    constexpr int STAGES = TSV_GEMM_STAGES;
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
    const int M = a.vp->m;  // asked for before the K loop, needed after it

    // Software pipeline over the K chunks, STAGES tiles in flight per wave.  Every load in the
    // steady state is unconditional (straight-line code), so the compiler can wait on the oldest
    // outstanding tile only (s_waitcnt vmcnt(n)) instead of draining the queue.
    if (nc > 0) {
        Stage<F, NG> st[STAGES];
        const ActLoader<false> x(a.xfrag, a.xsum, lane);
        const int last = c0 + nc - 1;
        auto fetch = [&](Stage<F, NG>& sg, int c) { load_stage(sg, x, wt + (size_t)c * F::TILE_BYTES, c, lane); };
#pragma unroll
        for (int s = 0; s < STAGES; s++) fetch(st[s], min(c0 + s, last));
        int c = 0;
        for (; c + 2 * STAGES <= nc; c += STAGES) {
#pragma unroll
            for (int s = 0; s < STAGES; s++) {
                compute(st[s], k, acc);
                fetch(st[s], c0 + c + s + STAGES);
            }
        }
        // last group that still has tiles to fetch (fewer than STAGES of them)
#pragma unroll
        for (int s = 0; s < STAGES; s++) {
            if (c + s < nc) {
                compute(st[s], k, acc);
                if (c + s + STAGES < nc) fetch(st[s], c0 + c + s + STAGES);
            }
        }
        c += STAGES;
#pragma unroll
        for (int s = 0; s < STAGES; s++)
            if (c + s < nc) compute(st[s], k, acc);
    }

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

// ------------------------------------------------------------------------------- nine to sixteen rows
// Passes of more than eight rows (draft trees, prompt blocks) over Q4_K weights run on
// v_mfma_f32_16x16x32_f16 instead: one instruction multiplies sixteen activation rows by sixteen
// weight rows over a whole 32-element sub-block, where the 4x4x4 form needs four row groups x
// eight K steps.  The tile bytes are the same; only the lane mapping differs:
//   lane (r, kg) = (lane % 16, lane / 16) of row block rb holds weight row 16 rb + r, elements
//   8 kg .. 8 kg + 7 of a sub-block (the B operand), and activation row r, same elements (the A
//   operand; rows past m multiply whatever the fragment buffer holds into output rows nobody
//   stores);  the result registers of the lane are activation rows 4 kg .. 4 kg + 3 of weight
//   row 16 rb + r.
// The two nibbles of a tile byte are the same element of sub-blocks 2p and 2p + 1, so one 8-byte
// load per (rb, p) feeds two MFMAs.  The code-offset / min term is one v_mfma_f32_16x16x4_f32 per
// four sub-blocks: lane (r, kg) supplies the sum of sub-block kg (kg + 4) of activation row r and
// the coefficient of weight row r for that sub-block.
typedef _Float16 half8 __attribute__((ext_vector_type(8)));

struct Stage16 {
    u32x2 q[4][4];  // [row block][sub-block pair]
    u32x4 h[4];     // scale header of the lane's weight row in each row block
    u32x2 x[8][2];  // [sub-block][K step] activation fragments
    float xs[2];    // activation sums of sub-blocks kg and kg + 4
};

__device__ __forceinline__ void load_stage16(Stage16& st, const GemmArgs& a, const uint8_t* tile_chunk, int c, int lane) {
    const int r = lane & 15, kg = lane >> 4;
    __builtin_amdgcn_sched_barrier(0);
    // fragment units (8 bytes) of chunk c: [64-element block][row group][K step][row in group]
    const u32x2* xp = (const u32x2*)a.xfrag + (size_t)c * 1024 + (r >> 2) * 64 + (r & 3) + kg * 8;
#pragma unroll
    for (int j = 0; j < 8; j++)
#pragma unroll
        for (int t = 0; t < 2; t++) st.x[j][t] = xp[(j >> 1) * 256 + ((j & 1) * 8 + t) * 4];
    const float* sp = a.xsum + (size_t)c * 128 + (r >> 2) * 32 + (r & 3) + kg * 4;
    st.xs[0] = sp[0];
    st.xs[1] = sp[16];
    const uint8_t* wp = tile_chunk + ((kg >> 1) * 64 + r) * 16 + (kg & 1) * 8;
#pragma unroll
    for (int rb = 0; rb < 4; rb++)
#pragma unroll
        for (int p = 0; p < 4; p++) st.q[rb][p] = __builtin_nontemporal_load((const u32x2*)(wp + (2 * p * 64 + 16 * rb) * 16));
#pragma unroll
    for (int rb = 0; rb < 4; rb++) st.h[rb] = __builtin_nontemporal_load((const u32x4*)(tile_chunk + 8192 + (16 * rb + r) * 16));
    __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ void compute16(const Stage16& st, const Consts& k, float4v (&acc)[4], int kg) {
    const float4v zero = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int rb = 0; rb < 4; rb++) {
        const u32x4 hs = st.h[rb];
        const float d = h2f_lo(hs.x), dmin = h2f_hi(hs.x);
        const uint32_t sl = hs.y & 0x3F3F3F3Fu, ml = hs.z & 0x3F3F3F3Fu;
        const uint32_t sh = (hs.w & 0x0F0F0F0Fu) | ((hs.y >> 2) & 0x30303030u);
        const uint32_t mh = ((hs.w >> 4) & 0x0F0F0F0Fu) | ((hs.z >> 2) & 0x30303030u);
        float sc[8];
#pragma unroll
        for (int j = 0; j < 8; j++) sc[j] = d * ubyte(j < 4 ? sl : sh, j & 3);
        // the lane's two coefficients of the offset term (sub-blocks kg and kg + 4 have kg's parity:
        // even ones carry the 1024 code offset, odd ones 64)
        const int sft = 8 * kg;
        const float off = (kg & 1) ? 64.0f : 1024.0f;
        const float cf_lo = -__builtin_fmaf(d * (float)((sl >> sft) & 0xFF), off, dmin * (float)((ml >> sft) & 0xFF));
        const float cf_hi = -__builtin_fmaf(d * (float)((sh >> sft) & 0xFF), off, dmin * (float)((mh >> sft) & 0xFF));
        float4v t = __builtin_amdgcn_mfma_f32_16x16x4f32(st.xs[0], cf_lo, zero, 0, 0, 0);
        t = __builtin_amdgcn_mfma_f32_16x16x4f32(st.xs[1], cf_hi, t, 0, 0, 0);
#pragma unroll
        for (int p = 0; p < 4; p++) {
            const u32x2 w = st.q[rb][p];
            const uint32_t w0 = w.x, w1 = w.x >> 8, w2 = w.y, w3 = w.y >> 8;
            const u32x4 blo = {and_or(w0, 0x000F000Fu, k.k6400), and_or(w1, 0x000F000Fu, k.k6400),
                               and_or(w2, 0x000F000Fu, k.k6400), and_or(w3, 0x000F000Fu, k.k6400)};
            const u32x4 bhi = {and_or(w0, 0x00F000F0u, k.k5400), and_or(w1, 0x00F000F0u, k.k5400),
                               and_or(w2, 0x00F000F0u, k.k5400), and_or(w3, 0x00F000F0u, k.k5400)};
            const u32x4 alo = {st.x[2 * p][0].x, st.x[2 * p][0].y, st.x[2 * p][1].x, st.x[2 * p][1].y};
            const u32x4 ahi = {st.x[2 * p + 1][0].x, st.x[2 * p + 1][0].y, st.x[2 * p + 1][1].x, st.x[2 * p + 1][1].y};
            const float4v dlo = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, alo),
                                                                       __builtin_bit_cast(half8, blo), zero, 0, 0, 0);
            const float4v dhi = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, ahi),
                                                                       __builtin_bit_cast(half8, bhi), zero, 0, 0, 0);
            fma4(t, sc[2 * p], dlo);
            fma4(t, sc[2 * p + 1], dhi);
        }
        acc[rb] += t;
    }
}

// v0 / v1: the finished sums of row blocks pr and pr + 2 (weight rows 16 pr + r and 32 + 16 pr + r of
// the tile); register i is activation row 4 kg + i.
template <int EPI>
__device__ __forceinline__ void epilogue16(const GemmArgs& a, int tile, int split, int pr, float4v v0, float4v v1,
                                           int lane, int M, float* ssum) {
    const int r = lane & 15, kg = lane >> 4;
    if (EPI == EPI_SILU) {
        // gate rows are the tile's first 32 rows, up rows the other 32: a lane holds both of a column
        const int col = tile * 32 + 16 * pr + r;  // K index of the down projection
        _Float16* out = (_Float16*)a.out;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const _Float16 h = pinned_half((_Float16)(silu_f(v0[i]) * v1[i]));
            float sum = (float)h;
#pragma unroll
            for (int o = 1; o < 16; o <<= 1) sum += __shfl_xor(sum, o);
            const int b = 4 * kg + i;
            if (b < M) out[a.out16 ? frag16_index(col, b) : frag_index(col, b)] = h;
            if (r == 0) ssum[pr * 16 + b] = sum;  // this half of the sub-block's sum
        }
        return;
    }
    if (EPI == EPI_ROPE) {
        const RopeEpi& e = a.rope;
        const int hd = e.hd, half = hd >> 1, tph = hd >> 6;
        const int tq = e.nq * tph, tk = e.nkv * tph;
        const int kind = tile < tq ? 0 : tile < tq + tk ? 1 : 2;
        const int st = kind == 0 ? tile : kind == 1 ? tile - tq : tile - tq - tk;
        const int head = st / tph, t = st - head * tph;
        const int idim = (tph == 2 ? 32 * t : 0) + 16 * pr + r;  // rotation pair index, 0 .. hd/2
        const int d0 = kind == 2 ? t * 64 + 16 * pr + r : idim, d1 = kind == 2 ? d0 + 32 : idim + half;
        const int sec = (kind == 0 ? 0 : kind == 1 ? e.nq * hd : (e.nq + e.nkv) * hd) + head * hd;
        const float b0 = e.bias ? e.bias[sec + d0] : 0.f, b1 = e.bias ? e.bias[sec + d1] : 0.f;
        const int base = a.vp->base;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int b = 4 * kg + i;
            if (b >= M) continue;
            const float x0 = v0[i] + b0, x1 = v1[i] + b1;
            float y0 = x0, y1 = x1;
            if (kind != 2) {
                const float2 cs = e.cs[b * half + idim];
                y0 = x0 * cs.x - x1 * cs.y;
                y1 = x0 * cs.y + x1 * cs.x;
            }
            const _Float16 h0 = (_Float16)y0, h1 = (_Float16)y1;
            if (kind == 0) {
                _Float16* q = (_Float16*)e.q16 + ((long)b * e.nq + head) * hd;
                q[d0] = h0;
                q[d1] = h1;
            } else {
                const int pos = (base + b) % e.max_ctx;
                if (kind == 1) {
                    ((_Float16*)e.kc)[kcache_index(head, pos, d0, hd, e.max_ctx)] = h0;
                    ((_Float16*)e.kc)[kcache_index(head, pos, d1, hd, e.max_ctx)] = h1;
                } else {
                    ((_Float16*)e.vc)[vcache_index(head, pos, d0, hd, e.max_ctx)] = h0;
                    ((_Float16*)e.vc)[vcache_index(head, pos, d1, hd, e.max_ctx)] = h1;
                }
            }
        }
        return;
    }
#pragma unroll
    for (int hf = 0; hf < 2; hf++) {
        const float4v v = hf ? v1 : v0;
        const int n = tile * 64 + 16 * (pr + 2 * hf) + r;
        if (n >= a.n_valid) continue;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const int b = 4 * kg + i;
            if (b >= M) continue;
            if (EPI == EPI_PARTIAL)
                ((float*)a.out)[((size_t)split * 16 + b) * a.ldo + n] = v[i];
            else
                ((_Float16*)a.out)[(size_t)b * a.ldo + n] = (_Float16)v[i];
        }
    }
}

template <int EPI>
__global__ __launch_bounds__(512) void k_gemm16(GemmArgs a) {
    extern __shared__ float4v red[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int split = blockIdx.x % a.splits, tile = blockIdx.x / a.splits;
    const int s0 = split * a.kslice, s1 = min(s0 + a.kslice, a.kchunks);
    const int c0 = min(s0 + wave * a.per, s1);
    const int nc = min(a.per, s1 - c0);
    const uint8_t* wt = a.w + (size_t)tile * a.kchunks * Q4K::TILE_BYTES;
    Consts k;
    k.k6400 = 0x64006400u;
    k.k5400 = 0x54005400u;
    k.k64 = 0x64646464u;
    asm volatile("" : "+v"(k.k6400), "+v"(k.k5400));
    float4v acc[4];
#pragma unroll
    for (int rb = 0; rb < 4; rb++) acc[rb] = float4v{0.f, 0.f, 0.f, 0.f};
    const int M = a.vp->m;
    if (nc > 0) {
        Stage16 st;
        load_stage16(st, a, wt + (size_t)c0 * Q4K::TILE_BYTES, c0, lane);
        for (int c = 1; c < nc; c++) {
            compute16(st, k, acc, lane >> 4);
            load_stage16(st, a, wt + (size_t)(c0 + c) * Q4K::TILE_BYTES, c0 + c, lane);
        }
        compute16(st, k, acc, lane >> 4);
    }
    // fold the waves' accumulators in wave order; wave w finishes the row-block pairs w, w + kparts
#pragma unroll
    for (int rb = 0; rb < 4; rb++) red[(wave * 4 + rb) * 64 + lane] = acc[rb];
    __syncthreads();
    float* ssum = (float*)(red + a.kparts * 256);
    for (int pr = wave; pr < 2; pr += a.kparts) {
        float4v v0 = red[pr * 64 + lane], v1 = red[(pr + 2) * 64 + lane];
        for (int w = 1; w < a.kparts; w++) {
            v0 += red[(w * 4 + pr) * 64 + lane];
            v1 += red[(w * 4 + pr + 2) * 64 + lane];
        }
        epilogue16<EPI>(a, tile, split, pr, v0, v1, lane, M, ssum);
    }
    if (EPI == EPI_SILU) {
        // a sub-block of the down projection is this tile's 32 columns: both halves' sums, then one store
        __syncthreads();
        if (threadIdx.x < 16 && (int)threadIdx.x < M) {
            float* sums = (float*)((char*)a.out + xfrag_sum_offset(a.n_valid));
            sums[xsum_index(tile, threadIdx.x)] = ssum[threadIdx.x] + ssum[16 + threadIdx.x];
        }
    }
}

// ------------------------------------------------------------------------------- prompt blocks of 64 rows
// A prompt pass of BLOCKS x 16 rows, here over Q4_K / Q5_K weights and further down over Q8_0, bf16 and Q6_K
// (crates/runtime/src/producer.rs:122-150: the chunked prefill runner feeds the prompt in blocks;
// families/llama/prefill.rs).  One workgroup per
// (tile, K slice), one wave per block of sixteen rows.  A tile chunk is unpacked ONCE per workgroup:
// wave w turns row block w of the chunk (sixteen weight rows x 256 K) into the B operands of
// v_mfma_f32_16x16x32_f16 and leaves them in LDS, in the lane order the 16-row kernel builds them in
// registers; after a barrier every wave multiplies all four row blocks by its own sixteen
// activation rows.  So the weight bytes, and the vector-ALU work of unpacking them, are spent once
// per 64 rows, and what is left per row block is matrix instructions.
// The activations come in the layout of frag16_index (a lane's sixteen bytes of a sub-block side by
// side: a wave's load is one contiguous KiB; the 16-row kernels' layout costs this kernel four times
// the bytes in partly used cache lines), which the producers of a prompt pass write on request.
//
// The unpacked operand is the integer sc_j * q (at most 63 * 15, exact in fp16), made from the
// offset codes by one packed fma: (1024 + q) * sc - 1024 * sc and (64 + q) * sc - 64 * sc are exact.
// With the sub-block scale inside the operand the eight sub-blocks of a chunk accumulate in one
// chain of matrix instructions, and the superblock scale d is applied once per chunk; the min term
// -dmin * m_j * sum_k x_k goes through v_mfma_f32_16x16x4_f32 as in the 16-row kernel.  The products
// are those of the same integers and the same fp16 activations as in the narrower kernels; only
// the order of the fp32 additions differs.
struct GemmWideArgs {
    GemmArgs g;         // block 0's view; blocks b > 0 sit at the strides below
    size_t x_stride;    // bytes between the blocks' activation fragments (sums included)
    size_t out_stride;  // bytes between the blocks' outputs (partial sums or fragments); unused by EPI_ROPE
    // g.vp: consecutive VerifyParams, one per block; g.rope.cs: [blocks * 16][hd / 2]; g.rope.q16: [blocks * 16][nq][hd]
};

constexpr int WIDE_BLOCKS = 4;
constexpr int WIDE_B_BYTES = 32768;             // [row block][sub-block pair][low / high nibbles][64 lanes][16 B]
constexpr int WIDE_BUF_BYTES = WIDE_B_BYTES + 4096;  // + [row block][64 lanes] (d, -dmin m_kg, -dmin m_(kg+4), 0)

struct WideW {  // what the unpacking wave holds of one chunk: its row block's codes and scale header
    u32x2 q[4];
    u32x4 h;
    u32x2 qh;  // Q5_K: the fifth bits of the lane's eight elements (bit 2 p / 2 p + 1 for pair p's low / high nibbles)
};
struct WideX {  // a block's activations of one chunk: the lane's A operand of every sub-block, and two sums
    u32x4 v[8];
    float xs[2];
};

// (the loads of a chunk stay where they are written, scheduling fences on both sides: left alone, the
// scheduler sinks them to their first use, one chunk later, and nothing is in flight ahead of the math)
template <bool Q5 = false>
__device__ __forceinline__ void wide_load_w(WideW& w, const uint8_t* tile_chunk, int rb, int lane) {
    const int r = lane & 15, kg = lane >> 4;
    const uint8_t* wp = tile_chunk + ((kg >> 1) * 64 + r) * 16 + (kg & 1) * 8;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int p = 0; p < 4; p++) w.q[p] = __builtin_nontemporal_load((const u32x2*)(wp + (2 * p * 64 + 16 * rb) * 16));
    w.h = __builtin_nontemporal_load((const u32x4*)(tile_chunk + 8192 + (16 * rb + r) * 16));
    if (Q5) w.qh = __builtin_nontemporal_load((const u32x2*)(wp + (9 * 64 + 16 * rb) * 16));  // units 9 and 10: byte l serves element l
    else w.qh = u32x2{0u, 0u};
    __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ void wide_load_x(WideX& x, const GemmArgs& a, int c, int lane) {
    const int r = lane & 15, kg = lane >> 4;
    const u32x4* xp = (const u32x4*)a.xfrag + (size_t)c * 512 + lane;  // frag16_index: [sub-block][lane][16 B]
    const float* sp = a.xsum + (size_t)c * 128 + (r >> 2) * 32 + (r & 3) + kg * 4;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 8; j++) x.v[j] = xp[j * 64];
    x.xs[0] = sp[0];
    x.xs[1] = sp[16];
    __builtin_amdgcn_sched_barrier(0);
}

// Row block `rb` of a chunk into LDS buffer `buf`.  Q5_K (q5_k.rs:47-96): the fifth bit of a code is OR-ed into the
// offset integer before the fma -- bit 4 of 1024 + q, bit 8 of the 1/16-ulp form of 64 + q -- and sc_j * q stays an
// exact fp16 integer (at most 63 * 31).
template <bool Q5 = false>
__device__ __forceinline__ void wide_unpack(const WideW& w, const Consts& k, uint8_t* buf, int rb, int lane) {
    typedef _Float16 half2v __attribute__((ext_vector_type(2)));
    const int kg = lane >> 4;
    const u32x4 hs = w.h;
    const float d = h2f_lo(hs.x), dmin = h2f_hi(hs.x);
    const uint32_t sl = hs.y & 0x3F3F3F3Fu, ml = hs.z & 0x3F3F3F3Fu;
    const uint32_t sh = (hs.w & 0x0F0F0F0Fu) | ((hs.y >> 2) & 0x30303030u);
    const uint32_t mh = ((hs.w >> 4) & 0x0F0F0F0Fu) | ((hs.z >> 2) & 0x30303030u);
    const int sft = 8 * kg;
    float4v coef;
    coef.x = d;
    coef.y = -(dmin * (float)((ml >> sft) & 0xFF));
    coef.z = -(dmin * (float)((mh >> sft) & 0xFF));
    coef.w = 0.f;
    *(float4v*)(buf + WIDE_B_BYTES + (rb * 64 + lane) * 16) = coef;
    const half2v m1024 = {(_Float16)-1024.0f, (_Float16)-1024.0f}, m64 = {(_Float16)-64.0f, (_Float16)-64.0f};
#pragma unroll
    for (int p = 0; p < 4; p++) {
        // the 6-bit scales of sub-blocks 2p (low nibbles) and 2p + 1 (high nibbles) as fp16 pairs
        const uint32_t s_lo = ((2 * p < 4 ? sl : sh) >> (8 * ((2 * p) & 3))) & 0xFFu;
        const uint32_t s_hi = ((2 * p + 1 < 4 ? sl : sh) >> (8 * ((2 * p + 1) & 3))) & 0xFFu;
        const half2v sc_lo = __builtin_bit_cast(half2v, k.k6400 | s_lo | (s_lo << 16)) + m1024;
        const half2v sc_hi = __builtin_bit_cast(half2v, k.k6400 | s_hi | (s_hi << 16)) + m1024;
        const half2v off_lo = sc_lo * m1024, off_hi = sc_hi * m64;
        const uint32_t w0 = w.q[p].x, w1 = w.q[p].x >> 8, w2 = w.q[p].y, w3 = w.q[p].y >> 8;
        const uint32_t wv[4] = {w0, w1, w2, w3};
        const uint32_t hv[4] = {w.qh.x, w.qh.x >> 8, w.qh.y, w.qh.y >> 8};
        u32x4 blo, bhi;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            uint32_t lo_bits = and_or(wv[i], 0x000F000Fu, k.k6400), hi_bits = and_or(wv[i], 0x00F000F0u, k.k5400);
            if (Q5) {
                const int slo = 4 - 2 * p;
                const uint32_t l5 = slo >= 0 ? hv[i] << (slo >= 0 ? slo : 0) : hv[i] >> (slo < 0 ? -slo : 0);
                lo_bits = and_or(l5, 0x00100010u, lo_bits);
                hi_bits = and_or(hv[i] << (7 - 2 * p), 0x01000100u, hi_bits);
            }
            const half2v lo = __builtin_bit_cast(half2v, lo_bits);  // 1024 + q
            const half2v hi = __builtin_bit_cast(half2v, hi_bits);  // 64 + q
            blo[i] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(lo, sc_lo, off_lo));
            bhi[i] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(hi, sc_hi, off_hi));
        }
        *(u32x4*)(buf + (((rb * 4 + p) * 2 + 0) * 64 + lane) * 16) = blo;
        *(u32x4*)(buf + (((rb * 4 + p) * 2 + 1) * 64 + lane) * 16) = bhi;
    }
}

// One chunk from LDS buffer `buf` against this wave's block.  The four row blocks are four independent
// accumulator chains, walked side by side (an activation operand is used four times in a row), and
// the operands of sub-block pair p + 1 are asked of LDS before the matrix instructions of pair p
// issue: a wave is alone on its SIMD here, so nothing else would cover the LDS latency.
__device__ __forceinline__ void wide_compute(const WideX& x, const uint8_t* buf, float4v (&acc)[4], int lane) {
    const float4v zero = {0.f, 0.f, 0.f, 0.f};
    float4v coef[4], t[4], tq[4];
    u32x4 blo[2][4], bhi[2][4];
    auto fetch = [&](int slot, int p) {
#pragma unroll
        for (int rb = 0; rb < 4; rb++) {
            blo[slot][rb] = *(const u32x4*)(buf + (((rb * 4 + p) * 2 + 0) * 64 + lane) * 16);
            bhi[slot][rb] = *(const u32x4*)(buf + (((rb * 4 + p) * 2 + 1) * 64 + lane) * 16);
        }
    };
#pragma unroll
    for (int rb = 0; rb < 4; rb++) coef[rb] = *(const float4v*)(buf + WIDE_B_BYTES + (rb * 64 + lane) * 16);
    fetch(0, 0);
#pragma unroll
    for (int rb = 0; rb < 4; rb++) {
        t[rb] = __builtin_amdgcn_mfma_f32_16x16x4f32(x.xs[0], coef[rb].y, zero, 0, 0, 0);
        tq[rb] = zero;
    }
#pragma unroll
    for (int rb = 0; rb < 4; rb++) t[rb] = __builtin_amdgcn_mfma_f32_16x16x4f32(x.xs[1], coef[rb].z, t[rb], 0, 0, 0);
#pragma unroll
    for (int p = 0; p < 4; p++) {
        if (p < 3) fetch((p + 1) & 1, p + 1);
        const u32x4 alo = x.v[2 * p], ahi = x.v[2 * p + 1];
#pragma unroll
        for (int rb = 0; rb < 4; rb++)
            tq[rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, alo), __builtin_bit_cast(half8, blo[p & 1][rb]),
                                                            tq[rb], 0, 0, 0);
#pragma unroll
        for (int rb = 0; rb < 4; rb++)
            tq[rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, ahi), __builtin_bit_cast(half8, bhi[p & 1][rb]),
                                                            tq[rb], 0, 0, 0);
    }
#pragma unroll
    for (int rb = 0; rb < 4; rb++) {
        fma4(t[rb], coef[rb].x, tq[rb]);
        acc[rb] += t[rb];
    }
}

// ---- the same pass over Q8_0 weights ---------------------------------------------------------
// A chunk is 128 K = four 32-element blocks, each with its own fp16 scale per weight row, so a block is
// one matrix instruction per row block whose result takes the block's scale in fp32 (fma4) on its way
// into the accumulator.  The operand is the signed code itself: the bytes become 1024 + (q + 128) by a
// byte permute against 0x64 as in the narrower kernel, and one packed add of -1152 -- exact -- leaves q;
// the activations' sums are not needed.  Products are again those of the same integers and the same
// fp16 activations as in the narrower kernels.
constexpr int WIDE80_B_BYTES = 16384;                    // [row block][block j][64 lanes][16 B]
constexpr int WIDE80_BUF_BYTES = WIDE80_B_BYTES + 4096;  // + [row block][64 lanes] the four scales as floats

struct WideW80 {
    u32x2 q[4];
    u32x2 d;
};
struct WideX80 {
    u32x4 v[4];
};

__device__ __forceinline__ void wide80_load_w(WideW80& w, const uint8_t* tile_chunk, int rb, int lane) {
    const int r = lane & 15, kg = lane >> 4;
    const uint8_t* wp = tile_chunk + ((kg >> 1) * 64 + 16 * rb + r) * 16 + (kg & 1) * 8;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 4; j++) w.q[j] = __builtin_nontemporal_load((const u32x2*)(wp + 2 * j * 64 * 16));
    w.d = __builtin_nontemporal_load((const u32x2*)(tile_chunk + 8192 + (16 * rb + r) * 8));
    __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ void wide80_load_x(WideX80& x, const GemmArgs& a, int c, int lane) {
    const u32x4* xp = (const u32x4*)a.xfrag + (size_t)c * 256 + lane;  // frag16_index: [block of 32 K][lane][16 B]
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 4; j++) x.v[j] = xp[j * 64];
    __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ void wide80_unpack(const WideW80& w, const Consts& k, uint8_t* buf, int rb, int lane) {
    typedef _Float16 half2v __attribute__((ext_vector_type(2)));
    const half2v off = {(_Float16)-1152.0f, (_Float16)-1152.0f};
    const float4v d = {h2f_lo(w.d.x), h2f_hi(w.d.x), h2f_lo(w.d.y), h2f_hi(w.d.y)};
    *(float4v*)(buf + WIDE80_B_BYTES + (rb * 64 + lane) * 16) = d;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const uint32_t wa = w.q[j].x ^ 0x80808080u, wb = w.q[j].y ^ 0x80808080u;
        const uint32_t sel[2] = {0x04020400u, 0x04030401u};  // bytes (0, 2) and (1, 3) under 0x64: 1024 + code
        u32x4 b;
#pragma unroll
        for (int i = 0; i < 2; i++) {
            b[i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2v, __builtin_amdgcn_perm(k.k64, wa, sel[i])) + off);
            b[2 + i] = __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2v, __builtin_amdgcn_perm(k.k64, wb, sel[i])) + off);
        }
        *(u32x4*)(buf + ((rb * 4 + j) * 64 + lane) * 16) = b;
    }
}

__device__ __forceinline__ void wide80_compute(const WideX80& x, const uint8_t* buf, float4v (&acc)[4], int lane) {
    const float4v zero = {0.f, 0.f, 0.f, 0.f};
    float4v d[4], t[4];
    u32x4 b[2][4];
    auto fetch = [&](int slot, int j) {
#pragma unroll
        for (int rb = 0; rb < 4; rb++) b[slot][rb] = *(const u32x4*)(buf + ((rb * 4 + j) * 64 + lane) * 16);
    };
#pragma unroll
    for (int rb = 0; rb < 4; rb++) d[rb] = *(const float4v*)(buf + WIDE80_B_BYTES + (rb * 64 + lane) * 16);
    fetch(0, 0);
#pragma unroll
    for (int j = 0; j < 4; j++) {
        if (j < 3) fetch((j + 1) & 1, j + 1);
#pragma unroll
        for (int rb = 0; rb < 4; rb++)
            t[rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, x.v[j]), __builtin_bit_cast(half8, b[j & 1][rb]),
                                                           zero, 0, 0, 0);
#pragma unroll
        for (int rb = 0; rb < 4; rb++) fma4(acc[rb], d[rb][j], t[rb]);
    }
}

// ---- the same pass over bf16 weights ---------------------------------------------------------
// A chunk is 64 K, and a tile's unit 4 s + kg already is what lane (r, kg) of v_mfma_f32_16x16x32_bf16
// holds of weight row r in K step s, so "unpacking" is a copy into LDS.  The fp16 activations go in as
// two bf16 terms, split exactly as in the narrower kernel (upper eight significant bits + remainder).
constexpr int WIDEBF_BUF_BYTES = 8192;  // [row block][K step][64 lanes][16 B]

struct WideWBf {
    u32x4 q[2];
};
struct WideXBf {
    u32x4 v[2];
};

__device__ __forceinline__ void widebf_load_w(WideWBf& w, const uint8_t* tile_chunk, int rb, int lane) {
    const int r = lane & 15, kg = lane >> 4;
    const uint8_t* wp = tile_chunk + (kg * 64 + 16 * rb + r) * 16;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int st = 0; st < 2; st++) w.q[st] = __builtin_nontemporal_load((const u32x4*)(wp + st * 4 * 64 * 16));
    __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ void widebf_load_x(WideXBf& x, const GemmArgs& a, int c, int lane) {
    const u32x4* xp = (const u32x4*)a.xfrag + (size_t)c * 128 + lane;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int st = 0; st < 2; st++) x.v[st] = xp[st * 64];
    __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ void widebf_store(const WideWBf& w, uint8_t* buf, int rb, int lane) {
#pragma unroll
    for (int st = 0; st < 2; st++) *(u32x4*)(buf + ((rb * 2 + st) * 64 + lane) * 16) = w.q[st];
}

__device__ __forceinline__ void widebf_compute(const WideXBf& x, const uint8_t* buf, float4v (&acc)[4], int lane) {
    typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
    u32x4 b[2][4];
#pragma unroll
    for (int st = 0; st < 2; st++)
#pragma unroll
        for (int rb = 0; rb < 4; rb++) b[st][rb] = *(const u32x4*)(buf + ((rb * 2 + st) * 64 + lane) * 16);
#pragma unroll
    for (int st = 0; st < 2; st++) {
        u32x4 hi, lo;
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const uint32_t word = x.v[st][i];
            const float f0 = h2f_lo(word), f1 = h2f_hi(word);
            const uint32_t b0 = __float_as_uint(f0) & 0xFFFF0000u, b1 = __float_as_uint(f1) & 0xFFFF0000u;
            const uint32_t r0 = __float_as_uint(f0 - __uint_as_float(b0)), r1 = __float_as_uint(f1 - __uint_as_float(b1));
            hi[i] = (b0 >> 16) | b1;
            lo[i] = (r0 >> 16) | (r1 & 0xFFFF0000u);
        }
#pragma unroll
        for (int rb = 0; rb < 4; rb++)
            acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, hi), __builtin_bit_cast(bf16x8, b[st][rb]),
                                                              acc[rb], 0, 0, 0);
#pragma unroll
        for (int rb = 0; rb < 4; rb++)
            acc[rb] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, lo), __builtin_bit_cast(bf16x8, b[st][rb]),
                                                              acc[rb], 0, 0, 0);
    }
}

// ---- the same pass over Q6_K weights ---------------------------------------------------------
// value = d * sc_j * (level - 32) with an int8 scale per 16 elements (crates/compute/src/quant_gguf/q6_k.rs:44-88).
// level - 32 is exact in fp16, but its product with the scale (up to 32 * 128) is not, so the scale goes in as
// sc = 16 a + b (a = sc >> 4 in -8..7, b = sc & 15): two operands (level - 32) * a and (level - 32) * b, both exact
// integers below 512, two chains of matrix instructions, and d * (16 * hi + lo) per 128 K in fp32.  A lane's eight
// K of a 32-K step lie inside one 16-element sub-block, so its scale is one byte.  The loop walks HALF chunks
// (128 K, two 64-K pairs): the two operands of a whole chunk would not leave room for two workgroups' buffers on a
// compute unit.  Lane (r, kg) finds its eight levels of step (pair p, half h) in word kg of unit 3 p + h (low
// nibbles: k0 k1 of the first 4-K step, k0 k1 of the second, then k2 k3, k2 k3) and in word 2 h + kg / 2 of unit
// 3 p + 2 (high bit pairs: extraction e = 4 (kg & 1) + 2 t + ab of 4-K step t in bits 2 e.. and 16 + 2 e..).
constexpr int WIDE6_B_BYTES = 32768;                   // [row block][32-K step of the half chunk][a / b][64 lanes][16 B]
constexpr int WIDE6_BUF_BYTES = WIDE6_B_BYTES + 1024;  // + [row block][64 lanes] d

struct WideW6 {
    uint32_t lo[2][2], hi[2][2];  // [pair of the half][h]
    u32x2 sc;                     // the half chunk's eight scales
    uint32_t d;
};
struct WideX6 {
    u32x4 v[4];
};

__device__ __forceinline__ void wide6_load_w(WideW6& w, const uint8_t* tile_chunk, int half, int rb, int lane) {
    const int r = lane & 15, kg = lane >> 4, row = 16 * rb + r;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int pp = 0; pp < 2; pp++) {
        const int p = 2 * half + pp;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            w.lo[pp][h] = __builtin_nontemporal_load((const uint32_t*)(tile_chunk + ((3 * p + h) * 64 + row) * 16 + 4 * kg));
            w.hi[pp][h] = __builtin_nontemporal_load((const uint32_t*)(tile_chunk + ((3 * p + 2) * 64 + row) * 16 + 4 * (2 * h + (kg >> 1))));
        }
    }
    w.sc = __builtin_nontemporal_load((const u32x2*)(tile_chunk + 12288 + row * 16 + 8 * half));
    w.d = __builtin_nontemporal_load((const uint32_t*)(tile_chunk + 13312 + row * 4));
    __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ void wide6_load_x(WideX6& x, const GemmArgs& a, int hc, int lane) {
    const u32x4* xp = (const u32x4*)a.xfrag + (size_t)hc * 256 + lane;  // frag16_index: four 32-K steps per half chunk
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int j = 0; j < 4; j++) x.v[j] = xp[j * 64];
    __builtin_amdgcn_sched_barrier(0);
}

__device__ __forceinline__ void wide6_unpack(const WideW6& w, const Consts& k, uint8_t* buf, int rb, int lane) {
    typedef _Float16 half2v __attribute__((ext_vector_type(2)));
    const int kg = lane >> 4;
    const half2v off = {(_Float16)-1056.0f, (_Float16)-1056.0f};
    *(float*)(buf + WIDE6_B_BYTES + (rb * 64 + lane) * 4) = h2f_lo(w.d);
#pragma unroll
    for (int pp = 0; pp < 2; pp++)
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const int sj = 4 * pp + 2 * h + (kg >> 1);  // the lane's sub-block among the half chunk's eight
            const uint32_t scw = sj < 4 ? w.sc.x : w.sc.y;
            const int sc8 = (int)(scw << (24 - 8 * (sj & 3))) >> 24;
            const _Float16 fa = (_Float16)(float)(sc8 >> 4), fb = (_Float16)(float)(sc8 & 15);
            const half2v a2 = {fa, fa}, b2 = {fb, fb};
            const uint32_t nw = w.lo[pp][h], H = w.hi[pp][h];
            u32x4 ba, bb;
#pragma unroll
            for (int t = 0; t < 2; t++)
#pragma unroll
                for (int ab = 0; ab < 2; ab++) {
                    const int e = 4 * (kg & 1) + 2 * t + ab;
                    const uint32_t lo = and_or(nw >> (8 * t + 4 * ab), 0x000F000Fu, k.k6400);
                    const uint32_t v = lo | (((H >> (2 * e)) << 4) & 0x00300030u);  // 1024 + level, twice
                    const half2v lv = __builtin_bit_cast(half2v, v) + off;             // level - 32
                    ba[2 * t + ab] = __builtin_bit_cast(uint32_t, lv * a2);
                    bb[2 * t + ab] = __builtin_bit_cast(uint32_t, lv * b2);
                }
            const int jj = 2 * pp + h;
            *(u32x4*)(buf + (((rb * 4 + jj) * 2 + 0) * 64 + lane) * 16) = ba;
            *(u32x4*)(buf + (((rb * 4 + jj) * 2 + 1) * 64 + lane) * 16) = bb;
        }
}

__device__ __forceinline__ void wide6_compute(const WideX6& x, const uint8_t* buf, float4v (&acc)[4], int lane) {
    const float4v zero = {0.f, 0.f, 0.f, 0.f};
    float d[4];
    float4v thi[4], tlo[4];
    u32x4 ba[2][4], bb[2][4];
    auto fetch = [&](int slot, int jj) {
#pragma unroll
        for (int rb = 0; rb < 4; rb++) {
            ba[slot][rb] = *(const u32x4*)(buf + (((rb * 4 + jj) * 2 + 0) * 64 + lane) * 16);
            bb[slot][rb] = *(const u32x4*)(buf + (((rb * 4 + jj) * 2 + 1) * 64 + lane) * 16);
        }
    };
#pragma unroll
    for (int rb = 0; rb < 4; rb++) {
        d[rb] = *(const float*)(buf + WIDE6_B_BYTES + (rb * 64 + lane) * 4);
        thi[rb] = zero;
        tlo[rb] = zero;
    }
    fetch(0, 0);
#pragma unroll
    for (int jj = 0; jj < 4; jj++) {
        if (jj < 3) fetch((jj + 1) & 1, jj + 1);
#pragma unroll
        for (int rb = 0; rb < 4; rb++)
            thi[rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, x.v[jj]), __builtin_bit_cast(half8, ba[jj & 1][rb]),
                                                             thi[rb], 0, 0, 0);
#pragma unroll
        for (int rb = 0; rb < 4; rb++)
            tlo[rb] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, x.v[jj]), __builtin_bit_cast(half8, bb[jj & 1][rb]),
                                                             tlo[rb], 0, 0, 0);
    }
#pragma unroll
    for (int rb = 0; rb < 4; rb++) {
        fma4(tlo[rb], 16.0f, thi[rb]);
        fma4(acc[rb], d[rb], tlo[rb]);
    }
}

// ---- the pass itself, whatever the storage type ------------------------------------------------
// What a storage type brings: its tile size, the size of an LDS buffer, how many loop units a K chunk
// makes (one; two half chunks for Q6_K), and the four steps of a unit -- load the unpacking wave's share of
// the tile, load a block's activations, unpack into LDS, multiply from LDS.
struct WideQ4 {
    static constexpr int TILE_BYTES = Q4K::TILE_BYTES, BUF_BYTES = WIDE_BUF_BYTES, UNITS = 1;
    typedef WideW W;
    typedef WideX X;
    static __device__ __forceinline__ void load_w(W& w, const uint8_t* t, int, int rb, int lane) { wide_load_w<false>(w, t, rb, lane); }
    static __device__ __forceinline__ void load_x(X& x, const GemmArgs& a, int u, int lane) { wide_load_x(x, a, u, lane); }
    static __device__ __forceinline__ void unpack(const W& w, const Consts& k, uint8_t* buf, int rb, int lane) { wide_unpack<false>(w, k, buf, rb, lane); }
    static __device__ __forceinline__ void compute(const X& x, const uint8_t* buf, float4v (&acc)[4], int lane) { wide_compute(x, buf, acc, lane); }
};
struct WideQ5 : WideQ4 {
    static constexpr int TILE_BYTES = Q5K::TILE_BYTES;
    static __device__ __forceinline__ void load_w(W& w, const uint8_t* t, int, int rb, int lane) { wide_load_w<true>(w, t, rb, lane); }
    static __device__ __forceinline__ void unpack(const W& w, const Consts& k, uint8_t* buf, int rb, int lane) { wide_unpack<true>(w, k, buf, rb, lane); }
};
struct WideQ8 {
    static constexpr int TILE_BYTES = Q80::TILE_BYTES, BUF_BYTES = WIDE80_BUF_BYTES, UNITS = 1;
    typedef WideW80 W;
    typedef WideX80 X;
    static __device__ __forceinline__ void load_w(W& w, const uint8_t* t, int, int rb, int lane) { wide80_load_w(w, t, rb, lane); }
    static __device__ __forceinline__ void load_x(X& x, const GemmArgs& a, int u, int lane) { wide80_load_x(x, a, u, lane); }
    static __device__ __forceinline__ void unpack(const W& w, const Consts& k, uint8_t* buf, int rb, int lane) { wide80_unpack(w, k, buf, rb, lane); }
    static __device__ __forceinline__ void compute(const X& x, const uint8_t* buf, float4v (&acc)[4], int lane) { wide80_compute(x, buf, acc, lane); }
};
struct WideBf {
    static constexpr int TILE_BYTES = BF16W::TILE_BYTES, BUF_BYTES = WIDEBF_BUF_BYTES, UNITS = 1;
    typedef WideWBf W;
    typedef WideXBf X;
    static __device__ __forceinline__ void load_w(W& w, const uint8_t* t, int, int rb, int lane) { widebf_load_w(w, t, rb, lane); }
    static __device__ __forceinline__ void load_x(X& x, const GemmArgs& a, int u, int lane) { widebf_load_x(x, a, u, lane); }
    static __device__ __forceinline__ void unpack(const W& w, const Consts&, uint8_t* buf, int rb, int lane) { widebf_store(w, buf, rb, lane); }
    static __device__ __forceinline__ void compute(const X& x, const uint8_t* buf, float4v (&acc)[4], int lane) { widebf_compute(x, buf, acc, lane); }
};
struct WideQ6 {
    static constexpr int TILE_BYTES = Q6K::TILE_BYTES, BUF_BYTES = WIDE6_BUF_BYTES, UNITS = 2;
    typedef WideW6 W;
    typedef WideX6 X;
    static __device__ __forceinline__ void load_w(W& w, const uint8_t* t, int half, int rb, int lane) { wide6_load_w(w, t, half, rb, lane); }
    static __device__ __forceinline__ void load_x(X& x, const GemmArgs& a, int u, int lane) { wide6_load_x(x, a, u, lane); }
    static __device__ __forceinline__ void unpack(const W& w, const Consts& k, uint8_t* buf, int rb, int lane) { wide6_unpack(w, k, buf, rb, lane); }
    static __device__ __forceinline__ void compute(const X& x, const uint8_t* buf, float4v (&acc)[4], int lane) { wide6_compute(x, buf, acc, lane); }
};

template <class P, int EPI>
__global__ __launch_bounds__(64 * WIDE_BLOCKS) void k_gemm_wide(GemmWideArgs wa) {
    extern __shared__ __attribute__((aligned(16))) uint8_t wide_lds[];  // two unit buffers, then the blocks' sub-block sums
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;  // wave = this wave's block = the row block it unpacks
    GemmArgs a = wa.g;
    a.xfrag = (const uint2*)((const uint8_t*)a.xfrag + (size_t)wave * wa.x_stride);
    a.xsum = (const float*)((const uint8_t*)a.xsum + (size_t)wave * wa.x_stride);
    a.out = a.out ? (uint8_t*)a.out + (size_t)wave * wa.out_stride : nullptr;
    a.vp = a.vp + wave;
    if (EPI == EPI_ROPE) {
        a.rope.cs += (size_t)wave * 16 * (a.rope.hd >> 1);
        a.rope.q16 += (size_t)wave * 16 * a.rope.nq * a.rope.hd;
    }
    const int split = blockIdx.x % a.splits, tile = blockIdx.x / a.splits;
    const int s0 = split * a.kslice, s1 = min(s0 + a.kslice, a.kchunks);
    const uint8_t* wt = a.w + (size_t)tile * a.kchunks * P::TILE_BYTES;
    Consts k;
    k.k6400 = 0x64006400u;
    k.k5400 = 0x54005400u;
    k.k64 = 0x64646464u;
    asm volatile("" : "+v"(k.k6400), "+v"(k.k5400), "+v"(k.k64));
    float4v acc[4];
#pragma unroll
    for (int rb = 0; rb < 4; rb++) acc[rb] = float4v{0.f, 0.f, 0.f, 0.f};
    const int M = a.vp->m;
    // unit u: unpack into buffer u & 1 -> ask for what comes next -> barrier -> multiply unit u.  The
    // barrier of unit u also separates the reads of unit u - 1 from the unpacking of unit u + 1,
    // which goes to the same buffer.  The codes are asked for two units ahead, the activations (which
    // come from L2) one.  No branch surrounds a load -- a unit index past the slice is clamped to its
    // last unit and that unit is simply asked for again -- so the loop body is one block and the
    // wait before each use is a count the compiler can know, not "everything".
    typename P::W w[2];
    typename P::X x[2];
    uint8_t* const buf0 = wide_lds;
    uint8_t* const buf1 = wide_lds + P::BUF_BYTES;
    const int u0 = P::UNITS * s0, u1 = P::UNITS * s1, last = u1 - 1;
    auto load_w = [&](typename P::W& ww, int u) {
        const int c = min(u, last);
        P::load_w(ww, wt + (size_t)(c / P::UNITS) * P::TILE_BYTES, c % P::UNITS, wave, lane);
    };
    load_w(w[0], u0);
    P::load_x(x[0], a, u0, lane);
    load_w(w[1], u0 + 1);
    int c = u0;
    for (; c + 2 <= u1; c += 2) {
        P::unpack(w[0], k, buf0, wave, lane);
        load_w(w[0], c + 2);
        P::load_x(x[1], a, min(c + 1, last), lane);
        __syncthreads();
        P::compute(x[0], buf0, acc, lane);
        P::unpack(w[1], k, buf1, wave, lane);
        load_w(w[1], c + 3);
        P::load_x(x[0], a, min(c + 2, last), lane);
        __syncthreads();
        P::compute(x[1], buf1, acc, lane);
    }
    if (c < u1) {
        P::unpack(w[0], k, buf0, wave, lane);
        __syncthreads();
        P::compute(x[0], buf0, acc, lane);
    }
    __syncthreads();  // every wave is done with the unit buffers before the epilogue's sums go to LDS behind them
    float* ssum = (float*)(wide_lds + 2 * P::BUF_BYTES) + wave * 32;
#pragma unroll
    for (int pr = 0; pr < 2; pr++) epilogue16<EPI>(a, tile, split, pr, acc[pr], acc[pr + 2], lane, M, ssum);
    if (EPI == EPI_SILU) {
        __syncthreads();
        if (lane < 16 && lane < M) {
            float* sums = (float*)((char*)a.out + xfrag_sum_offset(a.n_valid));
            sums[xsum_index(tile, lane)] = ssum[lane] + ssum[16 + lane];
        }
    }
}

// Fewest rows that go to the 16x16x32 form (TSV_GEMM16=0: never; TSV_GEMM16=<n>: from n rows on).
static int gemm16_min_rows() {
    static const int n = [] {
        const char* e = getenv("TSV_GEMM16");
        if (!e) return 9;
        const int v = atoi(e);
        return v <= 0 ? TSV_MAX_ROWS + 1 : v;
    }();
    return n;
}

static int launch16(hipStream_t s, const GemmArgs& a, int epi) {
    const size_t lds = (size_t)a.kparts * 4096 + 128;
    const dim3 grid(a.n_tiles * a.splits), block(64 * a.kparts);
    switch (epi) {
        case EPI_PARTIAL: hipLaunchKernelGGL(k_gemm16<EPI_PARTIAL>, grid, block, lds, s, a); break;
        case EPI_ROPE: hipLaunchKernelGGL(k_gemm16<EPI_ROPE>, grid, block, lds, s, a); break;
        case EPI_SILU: hipLaunchKernelGGL(k_gemm16<EPI_SILU>, grid, block, lds, s, a); break;
        default: hipLaunchKernelGGL(k_gemm16<EPI_LOGITS>, grid, block, lds, s, a); break;
    }
    TSV_HIP(hipGetLastError());
    return TSV_OK;
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
        case EPI_ROPE: return launch_e<F, EPI_ROPE>(s, a, m);
        case EPI_SILU: return launch_e<F, EPI_SILU>(s, a, m);
        default: return launch_e<F, EPI_LOGITS>(s, a, m);
    }
}

static int fill_gemm_args(GemmArgs& a, const TiledW& w, const uint4* xfrag, void* out, const VerifyParams* vp, int splits,
                          int epi, int ldo, int n_valid, const RopeEpi* rope) {
    if (epi != EPI_PARTIAL) splits = 1;
    if (splits < 1) splits = 1;
    if (splits > w.kchunks) splits = w.kchunks;
    a = GemmArgs{};
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
    if (epi == EPI_ROPE) {
        if (!rope || (rope->hd != 64 && rope->hd != 128) || w.n_rows != (rope->nq + 2 * rope->nkv) * rope->hd) {
            set_error("matmul: the rotating epilogue needs the fused q/k/v projection of a 64- or 128-wide head");
            return TSV_ERR_INVALID;
        }
        a.rope = *rope;
    }
    if (epi == EPI_SILU) {
        if (w.n_rows % 64) {
            set_error("matmul: gate/up rows must fill whole 64-row tiles");
            return TSV_ERR_INVALID;
        }
        a.n_valid = w.n_rows / 2;  // K of the next matmul
    }
    return TSV_OK;
}

int launch_gemm(hipStream_t s, const TiledW& w, const uint4* xfrag, void* out, const VerifyParams* vp,
                int m, int splits, int epi, int ldo, int n_valid, const RopeEpi* rope) {
    if (m < 1 || m > TSV_MAX_ROWS) {
        set_error("matmul: row count outside 1..16");
        return TSV_ERR_INVALID;
    }
    GemmArgs a;
    if (int rc = fill_gemm_args(a, w, xfrag, out, vp, splits, epi, ldo, n_valid, rope)) return rc;
    if (w.fmt == FMT_Q4K && m >= gemm16_min_rows()) return launch16(s, a, epi);
    return w.fmt == FMT_Q4K    ? launch_f<Q4K>(s, a, m, epi)
           : w.fmt == FMT_Q80  ? launch_f<Q80>(s, a, m, epi)
           : w.fmt == FMT_BF16 ? launch_f<BF16W>(s, a, m, epi)
           : w.fmt == FMT_Q6K  ? launch_f<Q6K>(s, a, m, epi)
           : w.fmt == FMT_Q5K  ? launch_f<Q5K>(s, a, m, epi)
                               : launch_f<MX4>(s, a, m, epi);
}

int gemm_wide_rows() { return 16 * WIDE_BLOCKS; }

// The same matmul over gemm_wide_rows() rows in blocks of sixteen: block b reads its fragments at
// xfrag + b * x_stride bytes, its parameters at vp + b, and writes at out + b * out_stride bytes
// (EPI_ROPE: rope->cs and rope->q16 hold all blocks' rows one after the other).  Q4_K, Q5_K, Q6_K, Q8_0 or bf16 weights.
template <class P, int EPI>
static int launch_wide_pe(hipStream_t s, const GemmWideArgs& wa) {
    const size_t lds = 2 * (size_t)P::BUF_BYTES + WIDE_BLOCKS * 32 * sizeof(float);
    static bool attr_set = false;  // more than 64 KiB of dynamic LDS has to be asked for once per kernel
    if (!attr_set && lds > 65536) {
        TSV_HIP(hipFuncSetAttribute((const void*)k_gemm_wide<P, EPI>, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        attr_set = true;
    }
    hipLaunchKernelGGL((k_gemm_wide<P, EPI>), dim3(wa.g.n_tiles * wa.g.splits), dim3(64 * WIDE_BLOCKS), lds, s, wa);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

template <class P>
static int launch_wide_p(hipStream_t s, const GemmWideArgs& wa, int epi) {
    switch (epi) {
        case EPI_PARTIAL: return launch_wide_pe<P, EPI_PARTIAL>(s, wa);
        case EPI_ROPE: return launch_wide_pe<P, EPI_ROPE>(s, wa);
        case EPI_SILU: return launch_wide_pe<P, EPI_SILU>(s, wa);
        default: set_error("matmul: prompt blocks have no logits epilogue"); return TSV_ERR_UNSUPPORTED;
    }
}

int launch_gemm_wide(hipStream_t s, const TiledW& w, const uint4* xfrag, size_t x_stride, void* out, size_t out_stride,
                     const VerifyParams* vp, int splits, int epi, int ldo, int n_valid, const RopeEpi* rope) {
    if (w.fmt != FMT_Q4K && w.fmt != FMT_Q5K && w.fmt != FMT_Q80 && w.fmt != FMT_BF16 && w.fmt != FMT_Q6K) {
        set_error("matmul: prompt blocks of 64 rows need Q4_K, Q5_K, Q6_K, Q8_0 or bf16 weights");
        return TSV_ERR_UNSUPPORTED;
    }
    GemmWideArgs wa{};
    if (int rc = fill_gemm_args(wa.g, w, xfrag, out, vp, splits, epi, ldo, n_valid, rope)) return rc;
    wa.x_stride = x_stride;
    wa.out_stride = out_stride;
    wa.g.out16 = 1;  // what this kernel reads is what it writes for the next one
    return w.fmt == FMT_Q4K    ? launch_wide_p<WideQ4>(s, wa, epi)
           : w.fmt == FMT_Q5K  ? launch_wide_p<WideQ5>(s, wa, epi)
           : w.fmt == FMT_Q80  ? launch_wide_p<WideQ8>(s, wa, epi)
           : w.fmt == FMT_BF16 ? launch_wide_p<WideBf>(s, wa, epi)
                               : launch_wide_p<WideQ6>(s, wa, epi);
}

}  // namespace tsv
