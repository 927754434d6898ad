// Routed-expert (MoE) FFN for a verify pass on gfx950.
//
// Replaces the reference's per-token expert dispatch (crates/runtime/src/families/llama/moe.rs,
// router semantics real_forward_dispatch.rs:1135-1158, expert math
// crates/gpu/src/shaders/moe_gguf.metal phase 1 / phase 2, CPU pattern crates/compute/src/moe.rs:22-73):
//   logits = router . x_norm;  top-k by logit, ties to the lower expert index;  softmax over the
//   selected logits only;  y = x + sum over slots IN RANK ORDER of w_slot * down_e(silu(gate_e x) * up_e x).
// Here all rows of the pass are routed at once and the experts are grouped: every expert that at
// least one row selected is multiplied ONCE, against just the rows that chose it (its weights are
// read once however many rows share it), by the same 64-row-tile MFMA sequences as the dense
// matmuls with a gathered activation operand.  The per-(row, slot) outputs are written apart and
// the next residual kernel adds them in slot order, so the sum has the reference's order.
#include <algorithm>
#include <cstdlib>

#include "gemm_core.h"

namespace tsv {

namespace {

// ---- router ---------------------------------------------------------------------------------
// One workgroup, one wave per row: the row's logits (split-K partials summed in order) sit
// 'ne / 64' per lane as order-preserving integer keys; k rounds of two wave-wide reductions on the
// DPP network (the largest key, then the lowest index that holds it: larger logit, then lower
// index) pick the experts in rank order.  Then one thread per (row, slot) pair finds the first
// pair that chose its expert -- the group's leader -- and its own place among that group's
// members, which are listed in pair order.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ uint32_t dpp_from(uint32_t v) {  // a lane without a source keeps its own value
    return (uint32_t)__builtin_amdgcn_update_dpp((int)v, (int)v, CTRL, ROW_MASK, 0xf, false);
}
// quad swaps, shifts by four and eight inside a row of sixteen, then the rows' last lanes handed
// on to the next row(s): lane 63 ends up with the reduction of all 64 (max and min are idempotent,
// so lanes that see a value twice do no harm)
__device__ __forceinline__ uint32_t wave_umax(uint32_t v) {
    v = max(v, dpp_from<0xb1, 0xf>(v));
    v = max(v, dpp_from<0x4e, 0xf>(v));
    v = max(v, dpp_from<0x114, 0xf>(v));
    v = max(v, dpp_from<0x118, 0xf>(v));
    v = max(v, dpp_from<0x142, 0xa>(v));
    v = max(v, dpp_from<0x143, 0xc>(v));
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}
__device__ __forceinline__ uint32_t wave_umin(uint32_t v) {
    v = min(v, dpp_from<0xb1, 0xf>(v));
    v = min(v, dpp_from<0x4e, 0xf>(v));
    v = min(v, dpp_from<0x114, 0xf>(v));
    v = min(v, dpp_from<0x118, 0xf>(v));
    v = min(v, dpp_from<0x142, 0xa>(v));
    v = min(v, dpp_from<0x143, 0xc>(v));
    return (uint32_t)__builtin_amdgcn_readlane((int)v, 63);
}
// float -> unsigned key with the same order (-0 is folded into +0 first, so equal floats have equal
// keys); key 0 is below every float's key and marks an expert that is taken or absent
__device__ __forceinline__ uint32_t order_key(float f) {
    const uint32_t u = __float_as_uint(f + 0.0f);
    return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key_value(uint32_t key) {
    return __uint_as_float((key & 0x80000000u) ? (key & 0x7FFFFFFFu) : ~key);
}

// The top-k of one row, by one wave: key[j] is the order key of expert lane + 64 j (0: absent).  Writes the row's
// weights and selections.
// `forced_first` / `forced_mine`: a.forced[m * 8] and a.forced[m * 8 + lane] (lane < k), asked for by the caller before its
// matmul so that they are not one more memory round trip here.
__device__ __forceinline__ void route_row(const MoeRouteArgs& a, int m, uint32_t (&key)[4], int lane, int forced_first,
                                          int forced_mine) {
    const int ne = a.n_experts, k = a.top_k;
    float top = 0.f, sum = 0.f, my_ex = 0.f;
    int my_sel = 0;
    const bool forced = forced_first >= 0;  // the same for the whole wave
    if (forced) {
        // lane r < k takes slot r's expert as given and fetches that expert's logit from the lane that holds it
        const int e = min(max(lane < k ? forced_mine : 0, 0), ne - 1);
        float l = 0.f;
#pragma unroll
        for (int j = 0; j < 4; j++) {
            const float v = __shfl(key_value(key[j]), e & 63);
            if ((e >> 6) == j) l = v;
        }
        top = key_value(wave_umax(lane < k ? order_key(l) : 0u));
        my_ex = expf(l - top);
        my_sel = e;
#pragma unroll
        for (int r = 0; r < 8; r++)
            if (r < k) sum += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_ex), r));
    }
#pragma unroll
    for (int r = 0; r < 8; r++) {
        if (r < k && !forced) {
            const uint32_t mine = max(max(key[0], key[1]), max(key[2], key[3]));
            const uint32_t kbest = wave_umax(mine);
            uint32_t idx = 0xFFFFFFFFu;  // ascending j is ascending index: the first maximum wins
#pragma unroll
            for (int j = 3; j >= 0; j--)
                if (key[j] == kbest) idx = (uint32_t)(lane + 64 * j);
            const int bi = (int)min(wave_umin(idx), (uint32_t)(ne - 1));
            const float best = key_value(kbest);
            if (r == 0) top = best;
            const float ex = expf(best - top);
            sum += ex;  // sequential in rank order, as `exps.iter().sum()`
            if (lane == r) {  // lane r keeps slot r
                my_ex = ex;
                my_sel = bi;
            }
#pragma unroll
            for (int j = 0; j < 4; j++)
                if (lane + 64 * j == bi) key[j] = 0;
        }
    }
    if (lane < k) {
        a.weights[m * 8 + lane] = my_ex / sum;
        a.selected[m * 8 + lane] = my_sel;
    }
}

// The ranking of every row of a pass: one workgroup, wave m ranks row m.  The router matmul before it is the dense
// one (split-K partial sums, a workgroup per tile and K slice): its sums are added here in split order.  The
// groups of rows that share an expert are not built here: every expert matmul workgroup derives its own from
// the selections (moe_derive_group), which takes a wave a few dozen instructions.
// (One launch for matmul and ranking -- a workgroup of sixteen waves per four rows walking the whole router --
// measured 12.3 us against 4.8 + 4.2 at 128 x 2048 Q8_0 and 19.5 against 4.6 + 4.3 at 128 x 2880 bf16: a
// workgroup's 32 or 90 tile chunks are issue-bound on its one compute unit.)
__global__ __launch_bounds__(1024) void k_route_rank(MoeRouteArgs a) {
    const int lane = threadIdx.x & 63, m = threadIdx.x >> 6;
    if (m >= a.m) return;
    if (a.blocks > 1) {  // a prompt pass: this workgroup's block of sixteen rows
        a.logits += (long)blockIdx.x * a.logits_block_stride;
        a.weights += blockIdx.x * 16 * 8;
        a.selected += blockIdx.x * 16 * 8;
        a.forced = nullptr;
    }
    const int ne = a.n_experts;
    // everything the row needs is asked for before the first add: the loads have no branch between them (a lane
    // past the last expert reads the last expert's, a split past the last split the last split's again)
    const int forced_first = a.forced ? a.forced[m * 8] : -1;
    const int forced_mine = a.forced ? a.forced[m * 8 + (lane & 7)] : -1;
    float part[4][8], bias[4];
    const int nj = ne <= 128 ? 2 : 4;
#pragma unroll
    for (int j = 0; j < 4; j++) {
        const int e = min(lane + 64 * j, ne - 1);
        bias[j] = a.bias && j < nj ? a.bias[e] : 0.f;  // before the top-k (families/gptoss/moe.rs:82-87)
#pragma unroll
        for (int sp = 0; sp < 8; sp++) part[j][sp] = j < nj ? a.logits[((size_t)min(sp, a.splits - 1) * 16 + m) * a.ld + e] : 0.f;
    }
    uint32_t key[4] = {0u, 0u, 0u, 0u};
#pragma unroll
    for (int j = 0; j < 4; j++) {
        float sum = 0.f;  // added in split order
#pragma unroll
        for (int sp = 0; sp < 8; sp++) sum += sp < a.splits ? part[j][sp] : 0.f;
        if (a.bias) sum += bias[j];
        if (j < nj && lane + 64 * j < ne) key[j] = order_key(sum);
    }
    route_row(a, m, key, lane, forced_first, forced_mine);
}

// ---- grouped expert matmul --------------------------------------------------------------------

__device__ __forceinline__ float silu_moe(float x) { return x / (1.0f + __expf(-x)); }

// One 64-row weight tile of expert `e` against up to four of the group's rows (r0 .. r0 + 3).
// STAGES: tiles in flight per wave.  Two when a wave has at most two K chunks to walk (both are then
// requested at once); one otherwise (90-100 VGPRs instead of 150-230, so twice the resident waves,
// which is worth more over a longer walk): the 120B-shaped step 5.86 -> 5.24 ms, the 30B-shaped one
// 4.43 ms either way.
// WIDE: the group is an expert's members among the 64 rows of a prompt pass (MoeGroupW): rows and members are
// addressed through their 16-row blocks, and every wave stays to the end so that the caller can go on to the
// group's next four members.
// NG: row groups of four walked side by side (the 64-row passes take four where an expert has many members: the
// tile is then unpacked once per sixteen rows instead of once per four).
template <class F, int EPI, int STAGES, bool WIDE = false, class G = MoeGroup, int NG = 1>
__device__ __forceinline__ void expert_tile(const MoeGemmArgs& a, const G& grp, int gi, int r0, float4v* red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, nw = blockDim.x >> 6;
    const int tile = blockIdx.x, e = grp.expert, cnt = grp.cnt;
    const int per = (a.kchunks + nw - 1) / nw;
    const int c0 = min(wave * per, a.kchunks), nc = min(per, a.kchunks - c0);
    const uint8_t* wt = a.w + ((size_t)e * a.tiles_per_expert + tile) * a.kchunks * F::TILE_BYTES;
    Consts k;
    k.k6400 = 0x64006400u;
    k.k5400 = 0x54005400u;
    k.k64 = 0x64646464u;
    asm volatile("" : "+v"(k.k6400), "+v"(k.k5400), "+v"(k.k64));

    // activation operand: gate/up gathers the pass's rows this expert was chosen by; down reads
    // the group's own buffer, whose rows are already in the group's order
    const uint8_t* xbase = (const uint8_t*)a.xfrag + (EPI == EPI_SLOT ? (size_t)gi * a.x_stride : 0);
    ActLoader<false> x(xbase, xbase + xfrag_sum_offset(a.k), lane);
#pragma unroll
    for (int g = 0; g < NG; g++) {
        const int mine = min(r0 + 4 * g + (lane & 3), cnt - 1);
        if (WIDE) {
            if (EPI == EPI_SILU) x.set_row_blocked(g, grp.rows[mine], a.x_block_stride);
            else x.set_row_blocked(g, mine, a.sub_stride);
        } else {
            x.set_row(g, EPI == EPI_SILU ? grp.rows[mine] : mine);
        }
    }

    float4v acc[NG];
#pragma unroll
    for (int g = 0; g < NG; g++) acc[g] = float4v{0.f, 0.f, 0.f, 0.f};
    if (nc > 0) {
        Stage<F, NG> st[STAGES];
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

    // fold the waves in wave order; wave 0 finishes
    __syncthreads();
#pragma unroll
    for (int g = 0; g < NG; g++) red[(wave * NG + g) * 64 + lane] = acc[g];
    __syncthreads();
    if (wave != 0) return;  // (WIDE: the caller's barrier is the next thing every wave meets)
#pragma unroll
    for (int g = 0; g < NG; g++) {
    const int rg = r0 + 4 * g;
    if (rg >= cnt) break;
    float4v v = red[g * 64 + lane];
    for (int w = 1; w < nw; w++) v += red[(w * NG + g) * 64 + lane];
    if (EPI == EPI_SILU) {
        // lanes 0..31: gate rows, lanes 32..63: up rows of the same 32 columns of this expert
        const int col = tile * 32 + (lane & 31);
        _Float16* out = (_Float16*)((uint8_t*)a.out + (size_t)gi * a.out_stride);
        float* sums = (float*)((uint8_t*)out + xfrag_sum_offset(a.n_out));
#pragma unroll
        for (int i = 0; i < 4; i++) {
            const float other = __shfl_xor(v[i], 32);
            float gate = lane < 32 ? v[i] : other, up = lane < 32 ? other : v[i];
            if (a.bias) {  // before the activation, where the clamp reads it too (moe_gguf.metal:585-600)
                gate += a.bias[(size_t)e * a.n_out + col];
                up += a.bias2[(size_t)e * a.n_out + col];
            }
            float act;
            if (a.alpha > 0.0f) {
                const float x = fminf(gate, a.limit), y = fminf(fmaxf(up, -a.limit), a.limit);
                act = (x / (1.0f + __expf(-a.alpha * x))) * (y + 1.0f);
            } else {
                act = silu_moe(gate) * up;
            }
            const _Float16 h = pinned_half((_Float16)act);
            float sum = (float)h;
#pragma unroll
            for (int o = 1; o < 32; o <<= 1) sum += __shfl_xor(sum, o);
            const int b = rg + i;  // the group's own row order
            if (b < cnt && lane < 32) {
                if (WIDE) {
                    _Float16* ow = (_Float16*)((uint8_t*)out + (size_t)(b >> 4) * a.sub_stride);
                    ow[frag_index(col, b & 15)] = h;
                    if (lane == 0) ((float*)((uint8_t*)ow + xfrag_sum_offset(a.n_out)))[xsum_index(col >> 5, b & 15)] = sum;
                } else {
                    out[frag_index(col, b)] = h;
                    if (lane == 0) sums[xsum_index(col >> 5, b)] = sum;
                }
            }
        }
    } else {
        const int n = tile * 64 + lane;
        if (n < a.n_out) {
#pragma unroll
            for (int i = 0; i < 4; i++) {
                const int b = rg + i;
                if (b < cnt) {
                    const int row = grp.rows[b];
                    const size_t at = WIDE ? (size_t)(row >> 4) * a.out_block_stride + ((size_t)grp.slots[b] * 16 + (row & 15)) * a.n_out
                                           : ((size_t)grp.slots[b] * 16 + row) * a.n_out;
                    ((float*)a.out)[at + n] = a.bias ? v[i] + a.bias[(size_t)e * a.n_out + n] : v[i];
                }
            }
        }
    }
    }
}

// grid: (tiles per expert, rows x top_k groups, sweeps).  Groups that repeat an earlier expert leave
// at once.  A workgroup multiplies its tile by four of the group's rows, 4 z .. 4 z + 3: an expert
// chosen by more than four rows is covered by several workgroups side by side, and those past the
// group's count leave at once.  With tiles x groups a multiple of eight the workgroups of one tile
// run on the same XCD, so the tile comes from HBM once and from that XCD's L2 after.
template <class F, int EPI, int STAGES>
__global__ __launch_bounds__(512) void k_moe_gemm(MoeGemmArgs a) {
    extern __shared__ float4v red[];
    __shared__ MoeGroup grp;
    const int gi = blockIdx.y, r0 = 4 * blockIdx.z;
    if (threadIdx.x < 64) moe_derive_group(&grp, a.selected, a.rows, a.top_k, gi, threadIdx.x);
    __syncthreads();
    if (r0 >= grp.cnt) return;
    expert_tile<F, EPI, STAGES>(a, grp, gi, r0, red);
}

// ---- the 64 rows of a prompt pass ---------------------------------------------------------------
// The members of every expert: one wave per expert walks the pass's (row, slot) pairs sixty-four at a time in
// pair order; a ballot marks the pairs that name the expert and a lane's place in the list is the count of
// marked pairs before it.  A row names an expert at most once, so a list has at most as many members as the
// pass has rows.
__global__ __launch_bounds__(1024) void k_moe_groups(const int32_t* __restrict__ selected, int rows, int top_k, int ne,
                                                     MoeGroupW* __restrict__ groups) {
    const int lane = threadIdx.x & 63, e = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
    if (e >= ne) return;
    MoeGroupW* g = groups + e;
    const int np = rows * top_k;
    int cnt = 0;
    for (int p0 = 0; p0 < np; p0 += 64) {
        const int p = p0 + lane;
        const int row = p / top_k, slot = p - row * top_k;
        const bool hit = p < np && selected[row * 8 + slot] == e;
        const uint64_t mask = __builtin_amdgcn_ballot_w64(hit);
        const int pos = cnt + __popcll(mask & ((1ull << lane) - 1ull));
        if (hit && pos < MOE_WIDE_ROWS) {
            g->rows[pos] = row;
            g->slots[pos] = slot;
        }
        cnt += __popcll(mask);
    }
    if (lane == 0) {
        g->expert = e;
        g->cnt = min(cnt, MOE_WIDE_ROWS);
    }
}

// grid: (tiles per expert, experts, 4).  Workgroup z takes the expert's members 4 z .. 4 z + 3, then sixteen further
// on, and so on: an expert few rows chose costs one workgroup per tile, one that many chose is spread over four.
// An expert with more than MOE_WIDE_HEAVY members is walked eight members at a time instead (workgroup z: members
// 8 z .. 8 z + 7, then 32 further on), so its tiles are unpacked half as often.
constexpr int MOE_WIDE_HEAVY = 8;
template <class F, int EPI, int STAGES>
__global__ __launch_bounds__(512) void k_moe_gemm_wide(MoeGemmArgs a) {
    extern __shared__ float4v red[];
    __shared__ MoeGroupW grp;
    const int e = blockIdx.y;
    const MoeGroupW* src = a.groups + e;
    const int cnt = min(src->cnt, MOE_WIDE_ROWS);
    if (4 * (int)blockIdx.z >= cnt) return;
    for (int i = threadIdx.x; i < MOE_WIDE_ROWS; i += blockDim.x) {
        grp.rows[i] = min(max(src->rows[min(i, cnt - 1)], 0), MOE_WIDE_ROWS - 1);
        grp.slots[i] = min(max(src->slots[min(i, cnt - 1)], 0), 7);
    }
    if (threadIdx.x == 0) {
        grp.expert = e;
        grp.cnt = cnt;
    }
    __syncthreads();
    if (cnt > MOE_WIDE_HEAVY) {
        // many members: eight per walk of the tile, one stage in flight (sixteen per walk costs 209 registers where this
        // costs 119-164, and the experts with few members, who share the kernel, lose their resident waves)
        for (int r0 = 8 * blockIdx.z; r0 < cnt; r0 += 8 * gridDim.z) {
            expert_tile<F, EPI, 1, true, MoeGroupW, 2>(a, grp, e, r0, red);
            __syncthreads();
        }
        return;
    }
    for (int r0 = 4 * blockIdx.z; r0 < cnt; r0 += 4 * gridDim.z) {
        expert_tile<F, EPI, STAGES, true, MoeGroupW, 1>(a, grp, e, r0, red);
        __syncthreads();
    }
}

template <class F, int EPI>
int launch_moe_wide_t(hipStream_t s, const MoeGemmArgs& a) {
    const int cpw = std::max(2, (a.kchunks + 3) / 4);
    const int nw = std::min(8, std::max(1, (a.kchunks + cpw - 1) / cpw));
    const size_t lds = (size_t)nw * 2 * 1024;  // two row groups' sums per wave
    const dim3 grid(a.tiles_per_expert, a.n_experts, 4);
    if ((a.kchunks + nw - 1) / nw <= 2)
        hipLaunchKernelGGL((k_moe_gemm_wide<F, EPI, 2>), grid, dim3(64 * nw), lds, s, a);
    else
        hipLaunchKernelGGL((k_moe_gemm_wide<F, EPI, 1>), grid, dim3(64 * nw), lds, s, a);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

template <int EPI>
int launch_moe_wide_f(hipStream_t s, int fmt, const MoeGemmArgs& a) {
    if (!a.groups || a.n_experts < 1 || a.n_experts > 256 || a.rows != MOE_WIDE_ROWS || a.x8_terms) {
        set_error("moe: a prompt pass lists its 64 rows' experts first and keeps fp16 activations");
        return TSV_ERR_INVALID;
    }
    return fmt == FMT_Q4K    ? launch_moe_wide_t<Q4K, EPI>(s, a)
           : fmt == FMT_Q80  ? launch_moe_wide_t<Q80, EPI>(s, a)
           : fmt == FMT_Q6K  ? launch_moe_wide_t<Q6K, EPI>(s, a)
           : fmt == FMT_Q5K  ? launch_moe_wide_t<Q5K, EPI>(s, a)
           : fmt == FMT_BF16 ? launch_moe_wide_t<BF16W, EPI>(s, a)
                             : launch_moe_wide_t<MX4, EPI>(s, a);
}

template <class F, int EPI>
int launch_moe_t(hipStream_t s, const MoeGemmArgs& a, int n_groups) {
    // waves per workgroup: about four, each with at least two K chunks of the tile to walk (measured on
    // the two routed configurations: 12 chunks -> 4 waves x 3, 8 chunks -> 4 x 2, 3 chunks -> 2 waves)
    static const int forced = [] {
        const char* e = getenv("TSV_MOE_CPW");
        return e ? std::max(1, atoi(e)) : 0;
    }();
    const int cpw = forced ? forced : std::max(2, (a.kchunks + 3) / 4);
    const int nw = std::min(8, std::max(1, (a.kchunks + cpw - 1) / cpw));
    const size_t lds = (size_t)nw * 1024;
    const dim3 grid(a.tiles_per_expert, n_groups, (std::max(1, a.rows) + 3) / 4);  // no group has more members than the pass has rows
    if ((a.kchunks + nw - 1) / nw <= 2)
        hipLaunchKernelGGL((k_moe_gemm<F, EPI, 2>), grid, dim3(64 * nw), lds, s, a);
    else
        hipLaunchKernelGGL((k_moe_gemm<F, EPI, 1>), grid, dim3(64 * nw), lds, s, a);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

template <int EPI>
int launch_moe_f(hipStream_t s, int fmt, const MoeGemmArgs& a, int n_groups) {
    return fmt == FMT_Q4K    ? launch_moe_t<Q4K, EPI>(s, a, n_groups)
           : fmt == FMT_Q80  ? launch_moe_t<Q80, EPI>(s, a, n_groups)
           : fmt == FMT_Q6K  ? launch_moe_t<Q6K, EPI>(s, a, n_groups)
           : fmt == FMT_Q5K  ? launch_moe_t<Q5K, EPI>(s, a, n_groups)
           : fmt == FMT_BF16 ? launch_moe_t<BF16W, EPI>(s, a, n_groups)
                             : launch_moe_t<MX4, EPI>(s, a, n_groups);
}

}  // namespace

int launch_route(hipStream_t s, const MoeRouteArgs& a) {
    if (a.n_experts > 256 || a.top_k < 1 || a.top_k > 8 || a.top_k > a.n_experts) {
        set_error("moe: at most 256 experts and top-k between 1 and 8");
        return TSV_ERR_UNSUPPORTED;
    }
    if (a.splits < 1 || a.splits > 8 || a.m < 1 || a.m > TSV_MAX_ROWS) {
        set_error("moe: the router's logits come in one to eight partial sums of at most sixteen rows");
        return TSV_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL(k_route_rank, dim3(std::max(1, a.blocks)), dim3(64 * a.m), 0, s, a);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

int launch_moe_groups(hipStream_t s, const int32_t* selected, int rows, int top_k, int n_experts, MoeGroupW* groups) {
    if (rows < 1 || rows > MOE_WIDE_ROWS || n_experts < 1 || n_experts > 256 || top_k < 1 || top_k > 8) {
        set_error("moe: at most 64 rows, 256 experts and top-k 8 in a prompt pass");
        return TSV_ERR_UNSUPPORTED;
    }
    hipLaunchKernelGGL(k_moe_groups, dim3((n_experts + 15) / 16), dim3(1024), 0, s, selected, rows, top_k, n_experts, groups);
    TSV_HIP(hipGetLastError());
    return TSV_OK;
}

int launch_moe_wide_gate_up(hipStream_t s, int fmt, const MoeGemmArgs& a) { return launch_moe_wide_f<EPI_SILU>(s, fmt, a); }

int launch_moe_wide_down(hipStream_t s, int fmt, const MoeGemmArgs& a) { return launch_moe_wide_f<EPI_SLOT>(s, fmt, a); }

int launch_moe_gate_up(hipStream_t s, int fmt, const MoeGemmArgs& a, int n_groups) {
    return launch_moe_f<EPI_SILU>(s, fmt, a, n_groups);
}

int launch_moe_down(hipStream_t s, int fmt, const MoeGemmArgs& a, int n_groups) {
    return launch_moe_f<EPI_SLOT>(s, fmt, a, n_groups);
}

}  // namespace tsv
