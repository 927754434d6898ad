// Internal declarations shared by the HIP translation units of libtsverify.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <string>
#include <vector>

#include "../../include/tsverify.h"
#include "../../include/tsverify_testing.h"

namespace tsv {

void set_error(const std::string& s);
bool error_is_empty();
const std::string& get_error();

#define TSV_HIP(call)                                                                       \
    do {                                                                                    \
        hipError_t e_ = (call);                                                             \
        if (e_ != hipSuccess) {                                                             \
            tsv::set_error(std::string(#call) + ": " + hipGetErrorString(e_));              \
            return TSV_ERR_DEVICE;                                                          \
        }                                                                                   \
    } while (0)

#define TSV_NEED(cond, msg)          \
    do {                             \
        if (!(cond)) {               \
            tsv::set_error(msg);     \
            return TSV_ERR_INVALID;  \
        }                            \
    } while (0)

// ---------------------------------------------------------------------------------------
// Device weight layout ("row tiles").  A matrix W[N][K] is cut into tiles of 64 output rows
// by one K-chunk (256 elements for Q4_K, 128 for Q8_0); tiles are stored [row tile][chunk]
// so a wave streaming along K for its 64 rows reads one contiguous byte run.  Lane l of the
// wave owns weight row l of the tile; every wave-wide load covers 1 KiB contiguous
// (64 lanes x 16 B):
//   Q4_K tile, 9216 B: [unit 0..7][lane][16 B] nibble bytes 16*unit.. of the lane's superblock,
//                      then [lane][16 B] (f16 d, f16 dmin, 12 packed scale bytes) -- the 144 B
//                      of each of the 64 superblocks, byte for byte, only re-ordered.
//   Q8_0 tile, 8704 B: [unit 0..7][lane][16 B] int8 quants (unit u = bytes 16*(u%2).. of block
//                      u/2 of the chunk), then [lane][4 x f16 d].
//   MXFP4 tile, 8704 B (64 rows x 256 K): [unit 0..7][lane][16 B] the 32 e2m1 nibbles of the
//                      lane's block u, nibbles re-ordered for the fp4 -> fp16 converter (see
//                      gemm_core.h), then [lane][8 e8m0 scale bytes].
//   Q6_K tile, 13568 B (64 rows x 256 K): per 64-K pair p three units [lane][16 B]: 3p and 3p + 1
//                      hold the low nibbles of K steps 0..7 / 8..15 (one word per two steps, nibble
//                      order k0 k1 of the first step, k0 k1 of the second, then k2 k3, k2 k3), 3p + 2
//                      the high bit pairs (one word per four steps: pair e in bits 2e.. is the first,
//                      pair e + 8 in bits 16 + 2e.. the second element of extraction e); then
//                      [lane][16 int8 scales], then [lane][f16 d + 2 B pad] -- the 210 bytes of a
//                      superblock, re-ordered.
//   bf16 tile, 8192 B (64 rows x 64 K): [unit 0..7][lane][16 B] the lane's row at K steps 2u and
//                      2u + 1, four values per step in the order k % 4 = 0, 2, 1, 3.
// Rows past the matrix's last row are all-zero blocks (scale 0).
//
// Activation layout ("fragments").  The <=16 fp16 activation rows of a K-wide matmul input
// are stored as the A operands of v_mfma_f32_4x4x4_16B_f16, ready to load one 8-byte word per
// lane: [K/64 pair][row group g = row/4][step b = (k%64)/4][i = row%4][4 halfs], the four halfs
// in the order the weight unpack produces (k%4 = 0, 2, 1, 3).  Behind the fragments
// (byte offset xfrag_sum_offset(K)) sit the fp32 sums of the fp16-rounded activations over
// every 32-element sub-block, [K/256][g][sub%8][i], which the matmul uses to take the
// integer-code offsets and the Q4_K min term back out.
// ---------------------------------------------------------------------------------------
enum { FMT_Q4K = 0, FMT_Q80 = 1, FMT_MX4 = 2, FMT_BF16 = 3, FMT_Q6K = 4, FMT_Q5K = 5 };

struct TiledW {
    uint8_t* tiles = nullptr;  // device
    int fmt = 0;
    int n_rows = 0;    // real output rows
    int n_tiles = 0;   // ceil(n_rows / 64)
    int kchunks = 0;   // K / chunk elems
    int k = 0;
    size_t bytes = 0;
};

inline int fmt_chunk_elems(int fmt) { return fmt == FMT_Q80 ? 128 : fmt == FMT_BF16 ? 64 : 256; }
inline int fmt_tile_bytes(int fmt) {
    return fmt == FMT_Q4K ? 9216 : fmt == FMT_Q5K ? 11264 : fmt == FMT_BF16 ? 8192 : fmt == FMT_Q6K ? 13568 : 8704;
}
inline int fmt_nsub(int fmt) { return fmt == FMT_Q80 ? 4 : fmt == FMT_BF16 ? 2 : fmt == FMT_Q6K ? 16 : 8; }
constexpr int TILE_ROWS = 64;

// An fp16 activation on its way to both the fragment store and the sub-block sum.  The matmuls multiply
// the sums by the weights' code offsets (up to 1024), so the sum must be that of the stored bits exactly;
// left alone, the compiler may convert the same fp32 value twice, with different instructions (a packed
// convert for the store, a fused multiply-convert for the sum).  Pinning the half in a register leaves it
// one copy to read.
__device__ __forceinline__ _Float16 pinned_half(_Float16 h) {
    uint32_t b = __builtin_bit_cast(uint16_t, h);
    asm volatile("" : "+v"(b));
    return __builtin_bit_cast(_Float16, (uint16_t)b);
}

// index (in halfs) of activation element (row, k) in the fragment layout
__host__ __device__ inline int frag_index(int k, int row) {
    const int pos = ((k & 1) << 1) | ((k >> 1) & 1);  // k%4 = 0,1,2,3 -> slot 0,2,1,3
    return ((((k >> 6) * 4 + (row >> 2)) * 16 + ((k >> 2) & 15)) * 4 + (row & 3)) * 4 + pos;
}
// The same activations as the 64-row prompt kernel reads them: [K / 32][K % 32 / 8][row][8 halfs], the sixteen
// bytes a lane of v_mfma_f32_16x16x32_f16 holds of its row, so a wave's load is one contiguous KiB.  Within
// every four K the halfs keep the order above; the sums sit behind, unchanged.
__host__ __device__ inline int frag16_index(int k, int row) {
    const int pos = ((k & 1) << 1) | ((k >> 1) & 1);
    return (((k >> 5) * 4 + ((k >> 3) & 3)) * 16 + row) * 8 + (k & 4) + pos;
}
// (K is rounded up to whole 256-element chunks: a matmul whose last chunk is only partly real
// reads zeros there, never the sums)
__host__ __device__ inline size_t xfrag_sum_offset(int k) { return (size_t)((k + 255) / 256) * 8192; }
__host__ __device__ inline size_t xfrag_bytes(int k) { return xfrag_sum_offset(k) + (size_t)((k + 255) / 256) * 512; }
// index (in floats) of the sum of sub-block `sub` (= k/32) of `row`
__host__ __device__ inline int xsum_index(int sub, int row) {
    return (((sub >> 3) * 4 + (row >> 2)) * 8 + (sub & 7)) * 4 + (row & 3);
}

// KV cache layouts (fp16).  Both caches are cut into blocks of 16 positions, and inside a block the halfs sit
// where the attention kernel's matrix instructions want them, so that every wave-wide load of that kernel is
// one contiguous KiB (64 lanes x 16 bytes):
//   K: [kv head][pos / 16][hd / 32][lane = 16 * ((d % 32) / 8) + pos % 16][8 halfs = d % 8] -- lane (j, kg) of
//      K step s holds dims 32 s + 8 kg .. + 7 of position j: the A operand of v_mfma_f32_16x16x32_f16;
//   V: [kv head][pos / 16][hd / 32][lane = 16 * ((pos % 16) / 4) + d % 16][(d / 16) % 2][4 halfs = pos % 4] -- the
//      A operands (V^T: dims x positions) of two v_mfma_f32_16x16x16_f16 output tiles side by side.
// `cap` is the number of positions the cache holds (a multiple of 16).
__host__ __device__ inline long kcache_index(int h, int pos, int d, int hd, int cap) {
    return (((long)h * (cap >> 4) + (pos >> 4)) * (hd >> 5) + (d >> 5)) * 512 + ((((d >> 3) & 3) * 16 + (pos & 15)) << 3) + (d & 7);
}
__host__ __device__ inline long vcache_index(int h, int pos, int d, int hd, int cap) {
    const int po = pos & 15;
    return (((long)h * (cap >> 4) + (pos >> 4)) * (hd >> 5) + (d >> 5)) * 512 +
           ((((po >> 2) * 16 + (d & 15)) * 2 + ((d >> 4) & 1)) << 2) + (po & 3);
}

// Per-call parameters every kernel of a verify pass reads from device memory, so a captured
// launch sequence can be replayed at another base position.
struct VerifyParams {
    int32_t m;               // rows of this pass
    int32_t base;            // position of row 0 == KV length before the pass
    int32_t feed[TSV_MAX_ROWS];
    int32_t pos[TSV_MAX_ROWS];   // rope position of row i: base + depth[i]
    uint32_t anc[TSV_MAX_ROWS];  // bit s set: row i attends cache slot base+s
};

enum { EPI_PARTIAL = 0, EPI_SILU = 1, EPI_LOGITS = 2, EPI_SLOT = 3, EPI_ROPE = 4 };

// What the fused q/k/v projection needs to finish its rows itself (EPI_ROPE): bias, NeoX rotation
// and the stores into the q buffer and the K / V cache slots.  The projection's rows are re-tiled
// so that the two halves of a rotation pair sit in lanes l and l + 32 of one tile.
struct RopeEpi {
    const float2* cs;    // [16][head_dim / 2] (cos, sin) of the rows' rotation angles, scaled
    const float* bias;   // nullable, fused q, k, v row order
    uint16_t* q16;       // [16][nq][hd] fp16
    uint16_t* kc;        // [nkv][max_ctx][hd]
    uint16_t* vc;        // [nkv][max_ctx/16][hd/16][64][4]
    int nq, nkv, hd, max_ctx;
};

struct GemmArgs {
    const uint8_t* w;
    const uint2* xfrag;  // activation fragments, 8 B per (pair, row group, lane)
    const float* xsum;   // their sub-block sums
    void* out;           // EPI_PARTIAL: float [splits][16][ldo]; EPI_SILU: fragments (+ sums) of the
                         // next matmul; EPI_LOGITS: half [m][ldo]
    const VerifyParams* vp;
    int n_tiles, kchunks, kslice, splits, kparts, per, ldo, n_valid;
    int out16;     // EPI_SILU: write the fragments in the prompt kernel's layout (frag16_index)
    RopeEpi rope;  // EPI_ROPE only
};

// Re-tiles n_rows GGUF rows of `raw` into `tiles`; source row r lands in tiled row
// (r / grp) * stride + offset + r % grp.
// (rowmap, when given, names the tiled row of every source row instead)
int launch_repack(hipStream_t s, int fmt, const uint8_t* raw, int n_rows, int k, uint8_t* tiles,
                  int kchunks, int grp, int stride, int offset, const int32_t* rowmap = nullptr);
int launch_gemm(hipStream_t s, const TiledW& w, const uint4* xfrag, void* out, const VerifyParams* vp,
                int m, int splits, int epi, int ldo, int n_valid, const RopeEpi* rope = nullptr);
int gemm_default_splits(const TiledW& w, int m);
// rows of a prompt-block pass, and the matmul over them in blocks of sixteen (Q4_K, Q5_K, Q6_K, Q8_0 or bf16 weights)
int gemm_wide_rows();
int launch_gemm_wide(hipStream_t s, const TiledW& w, const uint4* xfrag, size_t x_stride, void* out, size_t out_stride,
                     const VerifyParams* vp, int splits, int epi, int ldo, int n_valid, const RopeEpi* rope = nullptr);

// ---- routed experts (moe.hip) -----------------------------------------------------------------
// One routed expert of a pass: the rows that chose it (ascending) and the rank slot it has in
// each.  Groups are indexed by the (row, slot) pair at which the expert first appears; pairs that
// repeat an earlier expert hold cnt == 0, so a launch over rows x top_k groups touches every
// chosen expert exactly once and nothing else.
struct MoeGroup {
    int32_t expert, cnt;
    int32_t rows[16], slots[16];
};
// Prompt passes of 64 rows: the members of every expert, listed once per layer (k_moe_groups) -- the rows that chose
// it in pair order (row-major, then slot) and the slot it has in each.
constexpr int MOE_WIDE_ROWS = 64;
struct MoeGroupW {
    int32_t expert, cnt;
    int32_t rows[MOE_WIDE_ROWS], slots[MOE_WIDE_ROWS];
};
struct MoeRouteArgs {
    const float* logits;  // the router matmul's split-K partial sums: [splits][16][ld]
    int splits, ld;
    int n_experts, top_k;
    int m;              // rows of the pass (the launch sequence is per row count)
    float* weights;     // [16][8] softmax over the selected logits, rank order
    int32_t* selected;  // [16][8] expert ids, rank order
    const float* bias;  // nullable: n_experts values added to the logits before the top-k
    // nullable test hook: [16][8] expert ids a row is to take instead of its own top-k (slot order as
    // given, the weights still the softmax of the row's own logits over them); a row whose first
    // entry is negative routes freely
    const int32_t* forced;
    // a prompt pass of several 16-row blocks (one workgroup each): floats between the blocks' logits; weights and
    // selections of block b follow those of block b - 1; no forced routing
    int blocks;
    long logits_block_stride;
};
// The group of pair gi (row gi / k, slot gi % k) from the rows' selections, by one whole wave (lane = threadIdx.x
// < 64) into *g: the expert, the rows that chose it in pair order with the slot it has in each, and cnt != 0 only
// where pair gi is the first to name the expert.  Entries past the count repeat the last member, so a reader that
// takes entry n without looking at the count finds a row of the group.
__device__ __forceinline__ void moe_derive_group(MoeGroup* g, const int32_t* selected, int m, int k, int gi, int lane) {
    const int np = m * k, p0 = lane, p1 = lane + 64;
    const int e0 = p0 < np ? selected[(p0 / k) * 8 + p0 % k] : -1;
    const int e1 = p1 < np ? selected[(p1 / k) * 8 + p1 % k] : -2;
    const int ea = __builtin_amdgcn_readlane(e0, gi & 63), eb = __builtin_amdgcn_readlane(e1, gi & 63);
    const int e = gi < 64 ? ea : eb;
    const uint64_t m0 = __builtin_amdgcn_ballot_w64(e0 == e), m1 = __builtin_amdgcn_ballot_w64(e1 == e);
    const int c0 = __popcll(m0), cnt = c0 + __popcll(m1);
    const int first = m0 ? __ffsll((long long)m0) - 1 : 63 + __ffsll((long long)m1);
    const uint64_t below = (1ull << lane) - 1ull;
#pragma unroll
    for (int h = 0; h < 2; h++) {
        if ((h ? e1 : e0) != e) continue;
        const int p = h ? p1 : p0, pos = h ? c0 + __popcll(m1 & below) : __popcll(m0 & below);
        if (pos >= TSV_MAX_ROWS) continue;  // a row chooses an expert once: never more members than rows
        const int row = p / k, slot = p - row * k;
        g->rows[pos] = row;
        g->slots[pos] = slot;
        if (pos == cnt - 1)
            for (int q = cnt; q < TSV_MAX_ROWS; q++) {
                g->rows[q] = row;
                g->slots[q] = slot;
            }
    }
    if (lane == 0) {
        g->expert = e;
        g->cnt = first == gi ? min(cnt, TSV_MAX_ROWS) : 0;
    }
}
// Block-scaled fp8 activations: the B operand of the scaled-MFMA expert matmuls (MXFP4 experts).  A
// value is the sum of `terms` e4m3 numbers, each times the power-of-two scale of its 32-element
// block; term t holds what the terms before it left over, so three terms carry about 2^-13 of the
// block's largest element.  Byte i of word w of a block is element 4 w + {0, 2, 1, 3}[i]: the order
// of the weight tiles' nibbles.
struct X8 {
    uint8_t* q;  // [terms][16 rows][kpad] e4m3
    uint8_t* s;  // [terms][16 rows][kpad / 32] E8M0: scale = 2^(byte - 127)
    int kpad;    // K rounded up to whole 256-element chunks; the tail stays zero from the allocation
};
constexpr int X8_MAX_TERMS = 3;
// What a context uses unless TSV_MOE_FP4 says otherwise: 0, fp16 activations on the 4x4x4 MFMA (moe.hip).  The block-scaled
// fp8 operand of moe_fp4.hip is opt-in (TSV_MOE_FP4=2 or 3 terms): against the oracle at full depth, under the oracle's own
// routing, two terms came out 1.2e-2 of the logit range away at the Qwen3-30B-A3B configuration (48 layers) -- past the 1e-2
// the path is held to -- and 6.5e-3 at the gpt-oss-120B one; three terms 3.4e-3 / 4.2e-3; fp16 activations 5.5e-3 / 3.9e-3.
// Three terms cost what the instruction saves (gpt-oss-120B shape: 5.3 ms per step against 4.7), and where every row goes
// to its own experts the fp16 form is the fastest of the three.
constexpr int MOE_FP4_DEFAULT_TERMS = 0;
inline size_t x8_q_bytes(int k) { return (size_t)X8_MAX_TERMS * 16 * ((k + 255) / 256 * 256); }
inline size_t x8_s_bytes(int k) { return x8_q_bytes(k) / 32; }

struct MoeGemmArgs {
    const uint8_t* w;      // tiled weights of all experts, tiles_per_expert x kchunks tiles each
    int tiles_per_expert, kchunks, k;
    int rows;              // rows of the pass: the most members a group can have
    // scaled-MFMA path (x8_terms > 0, MXFP4 experts only): x8 replaces xfrag, o8 replaces the gate/up
    // output fragments; the strides are the bytes between the groups' buffers (0: one shared buffer)
    int x8_terms;
    X8 x8, o8;
    size_t x8_q_stride, x8_s_stride, o8_q_stride, o8_s_stride;
    const void* xfrag;     // gate/up: the pass's activation fragments; down: per-group fragments
    size_t x_stride;       // down: bytes between groups' fragment buffers
    void* out;             // gate/up: per-group fragments of silu(gate) * up; down: float [8 slots][16][n_out]
    size_t out_stride;
    int n_out;             // gate/up: expert FFN width; down: hidden
    const int32_t* selected;  // [rows][8] expert ids the rows chose (k_route_rank): the groups are derived from them
    int top_k;
    // nullable per-expert biases, [n_experts][n_out]: gate/up use bias (gate) and bias2 (up), added
    // before the activation; down uses bias, added before the slot is weighted
    const float* bias;
    const float* bias2;
    float alpha, limit;    // alpha > 0: clamped SwiGLU (moe_gguf.metal:528-556) instead of silu(g) * u
    // 64-row prompt passes (launch_moe_wide_*): one group per expert, listed in `groups`; a row r of the pass sits in
    // block r / 16 of the activation fragments and of the down outputs, member b of a group in sub-buffer b / 16 of
    // the group's own fragments
    const MoeGroupW* groups;
    int n_experts;
    size_t x_block_stride;    // gate/up: bytes between the blocks' activation fragments
    size_t sub_stride;        // bytes between the 16-member sub-buffers of a group's fragments
    size_t out_block_stride;  // down: floats between the blocks' [8 slots][16][n_out] outputs
};
int launch_route(hipStream_t s, const MoeRouteArgs& a);
int launch_moe_gate_up(hipStream_t s, int fmt, const MoeGemmArgs& a, int n_groups);
int launch_moe_down(hipStream_t s, int fmt, const MoeGemmArgs& a, int n_groups);
// the same two matmuls over the 64 rows of a prompt pass, and the listing of the experts' members before them
int launch_moe_groups(hipStream_t s, const int32_t* selected, int rows, int top_k, int n_experts, MoeGroupW* groups);
int launch_moe_wide_gate_up(hipStream_t s, int fmt, const MoeGemmArgs& a);
int launch_moe_wide_down(hipStream_t s, int fmt, const MoeGemmArgs& a);
// the same two matmuls on v_mfma_scale_f32_16x16x128_f8f6f4 (moe_fp4.hip)
int launch_moe_fp4_gate_up(hipStream_t s, const MoeGemmArgs& a, int n_groups);
int launch_moe_fp4_down(hipStream_t s, const MoeGemmArgs& a, int n_groups);

int launch_embed(hipStream_t s, const uint8_t* raw, int dtype, int hidden, float* x,
                 const VerifyParams* vp, int m, const float* freqs = nullptr, float mscale = 1.0f, int half = 0,
                 float2* cs = nullptr);
// Strides between the 16-row blocks of a prompt pass: rows and partial sums in floats, fragments in bytes.
struct NormBlocks {
    long x, partial, frag;
    int frag16;  // write the fragments in the prompt kernel's layout (frag16_index)
    void* frag2;  // nullable: a second fragment buffer (blocks `frag` bytes apart as well) that takes the other layout
};
// weights: NULL, or [16][8] factors of the partials (row m, partial s): the routed experts' sum
int launch_addnorm(hipStream_t s, float* x, const float* partial, int splits, int ldp, const float* w,
                   float eps, int hidden, uint4* xfrag, int m, const float* weights = nullptr,
                   const float* bias = nullptr, const X8* x8 = nullptr, int x8_terms = 0, int blocks = 1,
                   const NormBlocks* nb = nullptr);
int launch_f32_to_xfrag(hipStream_t s, const float* x, int k, uint4* xfrag, int m);
// the drafter head: fc's input rows as fragments (K = 2 * hidden) from the rows' next tokens (row 0's from device memory when
// token_dev is given) and residual rows; fills the rotation table, clears x_zero's rows
int launch_mtp_input(hipStream_t s, const uint8_t* raw, int dtype, const VerifyParams* vp, const int32_t* token_dev, int vocab,
                     const float* h_rows, const float* w_e, const float* w_t, const float* w_h, float eps, int hidden, uint4* xfrag,
                     float* x_zero, const float* freqs, float mscale, int half, float2* cs, int m);

struct RopeKvArgs {
    const float* qkv;  // [splits][16][ldq]
    int splits, ldq;
    const float* freqs;   // head_dim/2
    float mscale;         // multiplies cos and sin
    const float* bias;    // nullable: [ldq] projection biases in the fused q, k, v row order
    const float* q_norm;  // nullable, head_dim
    const float* k_norm;
    float eps;
    uint16_t* q16;  // [16][nq][hd] fp16
    uint16_t* kc;   // [nkv][max_ctx][hd]
    uint16_t* vc;   // [nkv][max_ctx/16][hd/16][64][4]
    int nq, nkv, hd, max_ctx;
    const VerifyParams* vp;
    // a prompt pass: `blocks` 16-row blocks (0 or 1: one), block b with parameters vp[b], partial sums qkv_block_stride
    // floats further on and its sixteen q rows behind block b - 1's
    int blocks;
    long qkv_block_stride;
    int paired;  // the q and k columns of a head come in the rotating epilogue's tile order (128-wide heads)
};
int launch_rope_kv(hipStream_t s, const RopeKvArgs& a, int m);

// The stores of a layer whose K / V rows are kept quantized (TurboQuant; layout in attn_tq_core.h)
struct TqKv {
    uint32_t* kq;   // [kv head][position][head_dim * k_bits / 32]
    float* kn;      // [kv head][position]
    uint32_t* vq;   // [kv head][position / 16][head_dim][1 or 2]
    float* vn;      // [kv head][position]
    const float* k_cb;  // codebook levels of the two sides
    const float* v_cb;
    int k_bits, v_bits;  // 0: the layer keeps fp16 rows
};

struct AttnArgs {
    const uint16_t* q16;
    const uint16_t* kc;
    const uint16_t* vc;
    float* part_o;   // [nkv][nch][rows][hd]
    float* part_ml;  // [nkv][nch][rows][2]
    uint4* xfrag;    // output, K index = qh*hd + d
    int nq, nkv, hd, max_ctx, nch;  // max_ctx: positions the layer's cache holds
    int ring;            // non-zero: the cache is a ring, position p in slot p % max_ctx (a windowed layer)
    float scale;
    int window;          // 0: full; else a row sees the last `window` positions of its sequence
    const float* sinks;  // nullable: one logit per q head joining the softmax maximum and denominator
    const VerifyParams* vp;
    // row count and base position by value when the launch knows them (saves the kernel one
    // dependent memory round trip before its first K/V load); base_hint < 0: read them from vp
    int m_hint, base_hint;
    int frag16;  // write the output fragments in the prompt kernel's layout (frag16_index)
    // nullable: head_dim signs.  The values were summed in a rotated space (a quantized KV layer); the merge
    // applies the normalized Hadamard transform to each head's result and multiplies by these signs
    // (crates/compute/src/kv_quant.rs:102-107) before it writes the fragments
    const float* unrot;
    TqKv tq;  // k_bits != 0: K and V come from these stores instead of kc / vc (q already rotated, unrot set)
    // a prompt pass of several 16-row blocks in one launch (blocks > 1): block b has its parameters at vp + b,
    // its base position at base_hint + 16 b, and its q rows, partial results and output fragments at the
    // strides below
    int blocks;
    // set by the launcher.  Non-zero: a one-dimensional grid in which the row groups of one (chunk, kv head) pair
    // take neighbouring slots of ONE of the eight dies (attn_grid_place), this many groups per pair
    int xcd_groups;
    size_t q_stride, part_o_stride, part_ml_stride;  // elements
    size_t frag_stride;                              // bytes
};
// Which (chunk, kv head, row group) a workgroup of the one-dimensional grid works on.  Workgroups go round the
// eight dies (XCDs, each with an L2 of its own) by linear index: index 8 s + x is slot s of die x.  A pair's row
// groups sit in slots next to each other on one die, so they start together and the K / V bytes the first one
// pulls in reach the others through that die's L2 instead of being fetched once per die.  False: a slot past the
// last pair, nothing to do.
__device__ inline bool attn_grid_place(const AttnArgs& a, int index, int& chunk, int& kvh, int& grp) {
    const int die = index & 7, slot = index >> 3;
    grp = slot % a.xcd_groups;
    const int pair = (slot / a.xcd_groups) * 8 + die;
    chunk = pair % a.nch;
    kvh = pair / a.nch;
    return pair < a.nch * a.nkv;
}
inline int attn_grid_size(int pairs, int groups) { return 8 * groups * ((pairs + 7) / 8); }
// the view of one block of such a launch
__host__ __device__ inline AttnArgs attn_block_view(const AttnArgs& a, int b) {
    AttnArgs v = a;
    v.q16 = a.q16 + (size_t)b * a.q_stride;
    v.part_o = a.part_o + (size_t)b * a.part_o_stride;
    v.part_ml = a.part_ml + (size_t)b * a.part_ml_stride;
    v.xfrag = (uint4*)((char*)a.xfrag + (size_t)b * a.frag_stride);
    v.vp = a.vp + b;
    if (a.base_hint >= 0) v.base_hint = a.base_hint + 16 * b;
    return v;
}
int launch_attention(hipStream_t s, const AttnArgs& a, int m);

// ---- quantized KV rows (kvquant.hip)
enum { TQ_TABLE_FLOATS = 512 + 16 + 16 };  // signs (head_dim <= 512), codebook and midpoints (<= 4 bits)
struct TqSide {
    const float* signs;  // head_dim
    const float* cb;     // 1 << bits
    const float* mid;    // (1 << bits) - 1
    int bits, words;     // packed words per row: ceil(head_dim * bits / 32)
};
struct TqArgs {
    uint16_t* q16;       // [m][nq][hd] fp16, rotated in place with the key signs
    // the pass's K / V rows as the q/k/v projection left them: fp16 caches of `stage_cap` positions in the
    // attention kernels' layouts, row b of the pass in slot (base + b) % stage_cap
    const uint16_t *kc, *vc;
    int stage_cap;
    TqKv store;          // where the rows go, at position base + b
    TqSide k, v;
    int nq, nkv, hd, cap;  // cap: positions the stores hold
    const VerifyParams* vp;
    int m_hint, base_hint;  // rows of the pass; position of its first row (< 0: read vp->base)
    float inv_sqrt2;        // set by the launcher
};
// words of a V group: the sixteen positions' indices of one dimension, 32 bits at two bits per index, else 64
__host__ __device__ constexpr int tq_v_group_words(int vb) { return vb == 2 ? 1 : 2; }
void tq_sign_vector(int dim, uint64_t seed, float* out);
std::vector<float> tq_codebook(int dim, int bits);
int tq_words(int hd, int bits);
int tq_upload_side(int hd, int bits, uint64_t seed, float* dev, TqSide* out);
// q rotation and quantization of the pass's rows into the stores
int launch_tq_prepare(hipStream_t s, const TqArgs& a);
// rows base + path[i] -> base + i of every quantized layer (stores_dev: one entry per layer, k_bits 0 where rows are fp16)
int launch_tq_gather(hipStream_t s, const TqKv* stores_dev, int n_layers, int nkv, int hd, int cap, const int32_t* path_dev, int n,
                     int base);
// bytes of a layer's four stores for `cap` positions (cap a multiple of 16)
size_t tq_kq_bytes(int nkv, int cap, int hd, int k_bits);
size_t tq_vq_bytes(int nkv, int cap, int hd, int v_bits);
int launch_attention_merge(hipStream_t s, const AttnArgs& a, int m);
int attn_chunks(int nkv);

int launch_kv_gather(hipStream_t s, uint16_t* const* caches_dev, const int32_t* caps_dev, int n_layers, int nkv, int hd,
                     const int32_t* path_dev, int n, int base);
int launch_kv_fill(hipStream_t s, uint16_t* kc, uint16_t* vc, int nkv, int hd, int max_ctx, int pos0, int n,
                   const uint16_t* k_in, const uint16_t* v_in);
int launch_kv_read(hipStream_t s, const uint16_t* kc, const uint16_t* vc, int nkv, int hd, int max_ctx,
                   int pos0, int n, uint16_t* k_out, uint16_t* v_out);

// ---- acceptance -------------------------------------------------------------------------
struct AcceptParams {
    int32_t m, k;            // rows, proposals (chain: m-1)
    int32_t vocab;
    int32_t tree;            // 0 chain, 1 tree
    int32_t sampled;
    int32_t n_stop;
    int32_t feed[TSV_MAX_ROWS];
    int32_t parent[TSV_MAX_ROWS];
    int32_t stop_tokens[16];
    double temperature;
    uint64_t seed, draw_step, generated, max_new_tokens;
    // truncation of the candidate set (crates/selection/src/choose.rs:111-228): 0 / false = off
    int32_t top_k, has_top_p, has_min_p, pad0;
    double top_p, min_p;
    // penalties (crates/selection/src/penalty.rs:15-82); pen == 0: none.  pen_cnt[v]: bit 31 = token v
    // is in the history, low bits = its occurrences in the generated suffix of the history.
    int32_t pen, pen_has_rep, pen_has_pf;
    float pen_rep;  // the repetition penalty as the clamped f32 the reference divides / multiplies by
    double pen_presence, pen_frequency;
    const uint32_t* pen_cnt;
};
struct AcceptResult {
    int32_t accepted, committed, next, stopped;
    uint64_t draw_step;
    int32_t path[TSV_MAX_ROWS + 1];
    int32_t path_len;
    double min_margin;
    int32_t error;  // 1: non-finite logit
};
struct AcceptScratch {
    double* stats;       // accept_stats_doubles() doubles: row statistics, partials, decisions
    double* work;        // [16 jobs][2][vocab] candidate masses (p, residual) + two more rows (tree residuals)
    uint64_t* hist;      // [16 jobs][2][65536] fixed-point mass per rank bin; a round clears what it uses first
    uint32_t* counters;  // ACCEPT_COUNTER_WORDS words: error flag, tree path, greedy arg-max partials
    uint64_t* tmass;     // [32 rows][65536] fixed-point softmax mass per rank bin (top-p cut)
    uint32_t* tcount;    // [32 rows][65536] candidates per rank bin (top-k / top-p cut)
    AcceptResult* result;  // device
};
constexpr int ACCEPT_COUNTER_WORDS = 1024;
size_t accept_stats_doubles();
// launches of the walk kernel a sampled tree round of this shape needs (parent[s] in [0, s), m <= TSV_MAX_ROWS)
int tree_walk_bound(const int32_t* parent, int m);
int launch_accept(hipStream_t s, const uint16_t* target, const uint16_t* draft, const AcceptParams* ap_dev,
                  const AcceptParams& ap_host, const AcceptScratch& sc);
int launch_draft_chain(hipStream_t s, const uint16_t* draft, const AcceptParams* ap_dev,
                       const AcceptParams& ap_host, const AcceptScratch& sc, int32_t* proposals_dev);
// arg-max of `rows` logit rows into out[0, rows); the error word (sc.counters[0]) is cleared first only on request
int launch_argmax_rows(hipStream_t s, const uint16_t* logits, int rows, int vocab, const AcceptScratch& sc, int32_t* out,
                       bool clear_error);
int noalloc_prepare_device();
}  // namespace tsv
// the library's own drafter head behind a tsv_drafter (NULL: someone else's), and its sampled block draft (runtime.hip)
tsv_ctx* tsv_mtp_own_head(const tsv_drafter* d);
int tsv_mtp_draft_block_sampled(tsv_ctx* head, int32_t anchor, int64_t base, int32_t block, const tsv_shaping* sh, uint64_t draw_step,
                                const int32_t* history, int64_t n_history, uint64_t generated, uint16_t* rows, int32_t* proposals);
namespace tsv {
int launch_pen_counts(hipStream_t s, const int32_t* history_dev, long n, long suffix_start, int vocab, uint32_t* cnt);

// ---- host utilities ----------------------------------------------------------------------
int64_t row_bytes(int dtype, int64_t cols);

}  // namespace tsv
