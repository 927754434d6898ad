// Routed-expert matmuls for MXFP4 experts on CDNA4's block-scaled matrix instruction
// (v_mfma_scale_f32_16x16x128_f8f6f4): the e2m1 codes and E8M0 block scales go to the matrix core as
// they sit in the weight tile, with no unpacking on the vector ALU, and one instruction multiplies
// 16 weight rows by up to 16 activation rows over 128 K, so an expert that many rows of the pass
// chose is still walked once.  Same routing, grouping, epilogues and summation order of the slots
// as moe.hip (reference: crates/runtime/src/families/llama/moe.rs, expert math
// crates/gpu/src/shaders/moe_gguf.metal phase 1 / phase 2, block format
// crates/compute/src/quant_gguf_mxfp4.rs:76-141).
//
// Operands.  A (weights, fp4): lane (r = lane % 16, g = lane / 16) of row block rb and K half h holds
// the 32 codes of block 4 h + g of tile row 16 rb + r -- one 16-byte unit of the tile -- and that
// block's scale byte.  B (activations, fp8 e4m3, struct X8): lane (n, g) holds row n's bytes
// [16 g, 16 g + 16) and [64 + 16 g, 64 + 16 g + 16) of the half's 128, and the scale byte of block
// 4 h + g (the instruction takes an 8-bit operand's K index as 64 (j / 16) + 16 g + j % 16 for byte j
// of the lane, a 4-bit operand's as 32 g + nibble, and every scale as that of K block g).  The
// activation bytes are stored in the element order of the tile's nibbles, so no operand is permuted
// here.  D: lane (n, g) holds activation row n against tile rows 16 rb + 4 g + {0..3}.
//
// The activations are split into TERMS fp8 terms (value = sum of terms, each with its own block
// scale), multiplied one after the other into the same accumulators.
#include <algorithm>
#include <cstdlib>

#include "gemm_core.h"
#include "x8.h"

namespace tsv {

namespace {

typedef int int8v __attribute__((ext_vector_type(8)));

constexpr int FP4_TILE = 8704;  // the MX4 tile: 8 units x 64 rows x 16 bytes of codes, then 8 scale bytes per row

template <int TERMS>
struct Fp4Stage {
    u32x4 w[4][2];         // [row block][K half]
    u32x2 ws[4];           // the eight scale bytes of the lane's row in each row block
    u32x4 x[TERMS][2][2];  // [term][K half][bytes 0..63 / 64..127 of the half]
    u32x2 xs[TERMS];       // the eight scale bytes of the lane's activation row
};

// Where a lane finds its activation row: byte offsets of the row inside a term's plane.
struct X8Row {
    const uint8_t* q;
    const uint8_t* s;
    size_t q_plane, s_plane;  // bytes between terms
};

template <int TERMS>
__device__ __forceinline__ void load_fp4(Fp4Stage<TERMS>& st, const uint8_t* tile, const X8Row& x, int c, int lane) {
    const int r = lane & 15, g = lane >> 4;
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < TERMS; t++) {
        const uint8_t* q = x.q + t * x.q_plane + c * 256 + g * 16;
#pragma unroll
        for (int h = 0; h < 2; h++) {
            st.x[t][h][0] = *(const u32x4*)(q + h * 128);
            st.x[t][h][1] = *(const u32x4*)(q + h * 128 + 64);
        }
        st.xs[t] = *(const u32x2*)(x.s + t * x.s_plane + c * 8);
    }
#pragma unroll
    for (int rb = 0; rb < 4; rb++) {
#pragma unroll
        for (int h = 0; h < 2; h++)
            st.w[rb][h] = __builtin_nontemporal_load((const u32x4*)(tile + ((4 * h + g) * 64 + 16 * rb + r) * 16));
        st.ws[rb] = __builtin_nontemporal_load((const u32x2*)(tile + 8192 + (16 * rb + r) * 8));
    }
    __builtin_amdgcn_sched_barrier(0);
}

template <int TERMS>
__device__ __forceinline__ void compute_fp4(const Fp4Stage<TERMS>& st, float4v (&acc)[4], int lane) {
    const int sh = (lane >> 4) * 8;  // the scale byte of K block g
    int sa[4][2];
#pragma unroll
    for (int rb = 0; rb < 4; rb++) {
        sa[rb][0] = (int)(st.ws[rb].x >> sh);
        sa[rb][1] = (int)(st.ws[rb].y >> sh);
    }
#pragma unroll
    for (int t = 0; t < TERMS; t++) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const u32x4 lo = st.x[t][h][0], hi = st.x[t][h][1];
            const int8v b = {(int)lo.x, (int)lo.y, (int)lo.z, (int)lo.w, (int)hi.x, (int)hi.y, (int)hi.z, (int)hi.w};
            const int sb = (int)((h ? st.xs[t].y : st.xs[t].x) >> sh);
#pragma unroll
            for (int rb = 0; rb < 4; rb++) {
                const u32x4 w = st.w[rb][h];
                const int8v a = {(int)w.x, (int)w.y, (int)w.z, (int)w.w, 0, 0, 0, 0};
                // A: fp4 (format 4), B: fp8 e4m3 (format 0); scales from byte 0 of the operands given
                acc[rb] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(a, b, acc[rb], 4, 0, 0, sa[rb][h], 0, sb);
            }
        }
    }
}

__device__ __forceinline__ float silu_fp4(float x) { return x / (1.0f + __expf(-x)); }

// grid: (tiles per expert, rows x top_k groups); groups that repeat an earlier expert leave at once.
// The waves of a workgroup split the tile's K chunks; wave 0 adds their sums in wave order and
// finishes the tile.
template <int EPI, int TERMS, int STAGES>
__global__ __launch_bounds__(512) void k_moe_fp4(MoeGemmArgs a) {
    extern __shared__ float4v red[];  // [waves - 1][4 row blocks][64 lanes]
    const int gi = blockIdx.y;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int n = lane & 15, g = lane >> 4;
    // the group of this workgroup's pair, derived from the rows' selections by the first wave.  Entries past the
    // group's count repeat its last member: such a lane multiplies that row again, from the same cache lines,
    // and its column of D is dropped.
    __shared__ MoeGroup grp_s;
    if (threadIdx.x < 64) moe_derive_group(&grp_s, a.selected, a.rows, a.top_k, gi, threadIdx.x);
    __syncthreads();
    const MoeGroup* grp = &grp_s;
    const int cnt = grp->cnt, e = grp->expert, my_row = grp->rows[n], my_slot = grp->slots[n];
    if (cnt == 0) return;
    const int tile = blockIdx.x;

    const int per = (a.kchunks + nw - 1) / nw;
    const int c0 = min(wave * per, a.kchunks), nc = min(per, a.kchunks - c0);
    const uint8_t* wt = a.w + ((size_t)e * a.tiles_per_expert + tile) * a.kchunks * FP4_TILE;

    // gate/up gathers the pass's rows this expert was chosen by; down reads the group's own buffer,
    // whose rows are in the group's order
    const int xrow = EPI == EPI_SILU ? my_row : min(n, cnt - 1);
    X8Row x;
    x.q_plane = (size_t)16 * a.x8.kpad;
    x.s_plane = (size_t)16 * (a.x8.kpad >> 5);
    x.q = a.x8.q + (size_t)gi * a.x8_q_stride + (size_t)xrow * a.x8.kpad;
    x.s = a.x8.s + (size_t)gi * a.x8_s_stride + (size_t)xrow * (a.x8.kpad >> 5);

    float4v acc[4];
#pragma unroll
    for (int rb = 0; rb < 4; rb++) acc[rb] = float4v{0.f, 0.f, 0.f, 0.f};
    if (nc > 0) {
        Fp4Stage<TERMS> st[STAGES];
        const int last = c0 + nc - 1;
        auto fetch = [&](Fp4Stage<TERMS>& sg, int c) { load_fp4(sg, wt + (size_t)c * FP4_TILE, x, c, lane); };
#pragma unroll
        for (int s = 0; s < STAGES; s++) fetch(st[s], min(c0 + s, last));
        int c = 0;
        for (; c + 2 * STAGES <= nc; c += STAGES) {
#pragma unroll
            for (int s = 0; s < STAGES; s++) {
                compute_fp4(st[s], acc, lane);
                fetch(st[s], c0 + c + s + STAGES);
            }
        }
#pragma unroll
        for (int s = 0; s < STAGES; s++) {
            if (c + s < nc) {
                compute_fp4(st[s], acc, lane);
                if (c + s + STAGES < nc) fetch(st[s], c0 + c + s + STAGES);
            }
        }
        c += STAGES;
#pragma unroll
        for (int s = 0; s < STAGES; s++)
            if (c + s < nc) compute_fp4(st[s], acc, lane);
    }

    float4v v[4];
    if (nw > 1) {
        if (wave != 0) {
#pragma unroll
            for (int rb = 0; rb < 4; rb++) red[((wave - 1) * 4 + rb) * 64 + lane] = acc[rb];
        }
        __syncthreads();
        if (wave != 0) return;
#pragma unroll
        for (int rb = 0; rb < 4; rb++) {
            v[rb] = acc[rb];
            for (int w = 1; w < nw; w++) v[rb] += red[((w - 1) * 4 + rb) * 64 + lane];
        }
    } else {
#pragma unroll
        for (int rb = 0; rb < 4; rb++) v[rb] = acc[rb];
    }

    if (EPI == EPI_SILU) {
        // tile rows 0..31 are gate, 32..63 up, of the same 32 columns: row blocks (0, 2) and (1, 3) pair
        // up inside the lane.  The 32 columns are one block of the down matmul's K axis.
        const int col0 = tile * 32 + 4 * g;  // + 16 rb + i
        float act[2][4];
#pragma unroll
        for (int rb = 0; rb < 2; rb++) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                float gate = v[rb][i], up = v[rb + 2][i];
                const int col = col0 + 16 * rb + i;
                if (a.bias) {  // before the activation, where the clamp reads it too (moe_gguf.metal:585-600)
                    gate += a.bias[(size_t)e * a.n_out + col];
                    up += a.bias2[(size_t)e * a.n_out + col];
                }
                if (a.alpha > 0.0f) {
                    const float xg = fminf(gate, a.limit), y = fminf(fmaxf(up, -a.limit), a.limit);
                    act[rb][i] = (xg / (1.0f + __expf(-a.alpha * xg))) * (y + 1.0f);
                } else {
                    act[rb][i] = silu_fp4(gate) * up;
                }
            }
        }
        // stored order of a word: elements (0, 2, 1, 3)
        float r0[4] = {act[0][0], act[0][2], act[0][1], act[0][3]}, r1[4] = {act[1][0], act[1][2], act[1][1], act[1][3]};
        uint8_t* oq = a.o8.q + (size_t)gi * a.o8_q_stride + (size_t)n * a.o8.kpad + tile * 32 + 4 * g;
        uint8_t* os = a.o8.s + (size_t)gi * a.o8_s_stride + (size_t)n * (a.o8.kpad >> 5) + tile;
#pragma unroll
        for (int t = 0; t < TERMS; t++) {
            float amax = fmaxf(x8_amax4(r0), x8_amax4(r1));
            amax = fmaxf(amax, __shfl_xor(amax, 16));
            amax = fmaxf(amax, __shfl_xor(amax, 32));
            const int byte = x8_scale_byte(amax);
            const uint32_t w0 = x8_term4(r0, byte), w1 = x8_term4(r1, byte);
            if (n < cnt) {
                *(uint32_t*)(oq + (size_t)t * 16 * a.o8.kpad) = w0;
                *(uint32_t*)(oq + (size_t)t * 16 * a.o8.kpad + 16) = w1;
                if (g == 0) os[(size_t)t * 16 * (a.o8.kpad >> 5)] = (uint8_t)byte;
            }
        }
    } else {
        if (n < cnt) {
            float* out = (float*)a.out + ((size_t)my_slot * 16 + my_row) * a.n_out + tile * 64 + 4 * g;
#pragma unroll
            for (int rb = 0; rb < 4; rb++) {
                float4v o = v[rb];
                if (a.bias) {
                    const float4v b = *(const float4v*)(a.bias + (size_t)e * a.n_out + tile * 64 + 16 * rb + 4 * g);
                    o += b;
                }
                *(float4v*)(out + 16 * rb) = o;
            }
        }
    }
}

template <int EPI, int TERMS>
int launch_fp4_t(hipStream_t s, const MoeGemmArgs& a, int n_groups) {
    // About four waves on a tile (measured at 3, 8 and 12 chunks, with few and with many experts in
    // play: 3 x 1, 4 x 2 and 4 x 3 beat both more, shorter waves -- whose sums wave 0 then folds alone
    // -- and fewer, longer ones).  One register stage: a second stage in flight (227 VGPRs against
    // 124) halves the resident waves and measured slower at every shape, also where a wave has exactly two chunks to walk.  TSV_MOE_FP4_CPW: chunks per wave.
    static const int forced = [] {
        const char* e = getenv("TSV_MOE_FP4_CPW");
        return e ? std::max(1, atoi(e)) : 0;
    }();
    const int cpw = forced ? forced : (a.kchunks + 3) / 4;
    const int nw = std::min(8, std::max(1, (a.kchunks + cpw - 1) / cpw));
    const size_t lds = (size_t)std::max(1, nw - 1) * 4 * 1024;
    hipLaunchKernelGGL((k_moe_fp4<EPI, TERMS, 1>), dim3(a.tiles_per_expert, n_groups), dim3(64 * nw), lds, s, a);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

template <int EPI>
int launch_fp4(hipStream_t s, const MoeGemmArgs& a, int n_groups) {
    if (!a.x8.q || !a.x8.s || a.x8.kpad != a.kchunks * 256 || (EPI == EPI_SILU && (!a.o8.q || !a.o8.s || a.o8.kpad < a.n_out))) {
        set_error("moe (scaled MFMA): activation buffers do not match the matmul's K");
        return TSV_ERR_INVALID;
    }
    if (EPI == EPI_SLOT && a.n_out != a.tiles_per_expert * 64) {
        set_error("moe (scaled MFMA): the down matmul's width must be whole 64-row tiles");
        return TSV_ERR_INVALID;
    }
    switch (a.x8_terms) {
        case 2: return launch_fp4_t<EPI, 2>(s, a, n_groups);
        case 3: return launch_fp4_t<EPI, 3>(s, a, n_groups);
        default: set_error("moe (scaled MFMA): two or three activation terms"); return TSV_ERR_INVALID;
    }
}

}  // namespace

int launch_moe_fp4_gate_up(hipStream_t s, const MoeGemmArgs& a, int n_groups) { return launch_fp4<EPI_SILU>(s, a, n_groups); }
int launch_moe_fp4_down(hipStream_t s, const MoeGemmArgs& a, int n_groups) { return launch_fp4<EPI_SLOT>(s, a, n_groups); }

}  // namespace tsv
