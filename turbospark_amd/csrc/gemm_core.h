// Device-side core of the dequant-fused small-M matmul: weight-tile formats, the register stage
// of the software pipeline, and the per-tile MFMA sequences.  Shared by the stand-alone matmul
// kernel and the fused per-XCD layer kernels.
#pragma once
#include <utility>

#include "tsv_internal.h"

namespace tsv {

typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

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

typedef __attribute__((address_space(3))) void* lds_ptr;

// 32-bit LDS address of a generic pointer into shared memory
__device__ __forceinline__ uint32_t lds_addr(const void* p) {
    return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const void*)p;
}

// One wave-wide global -> LDS transfer, 16 (or 4) bytes per lane to lds + lane * size, done by the
// memory pipeline without passing through registers; vmcnt counts it like a load.  Written as
// inline assembly on purpose: the compiler then neither sees an LDS write (it would otherwise
// drain the whole load queue before the next LDS access) nor counts the transfer, which only
// makes its own s_waitcnt values wait for a few more, older, operations.  Readers of the
// buffer order themselves after a later load with lds_after().
__device__ __forceinline__ void dma_to_lds_b128(const void* g, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds), "v"(g) : "memory");
}
__device__ __forceinline__ void dma_to_lds_b32(const void* g, uint32_t lds) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, off" ::"s"(lds), "v"(g) : "memory");
}
// An LDS address the compiler believes to depend on `loaded`, a register filled by a load that
// was issued after the transfers into that buffer: loads complete in issue order, so once the
// compiler has waited for `loaded`, the buffer is complete, and no read through the returned
// address can be scheduled before that wait.
__device__ __forceinline__ uint32_t lds_after(uint32_t lds, float loaded) {
    asm volatile("" : "+v"(lds) : "v"(loaded));
    return lds;
}

// ------------------------------------------------------------------------------- formats
struct Q4K {
    static constexpr int NSUB = 8, NPAIR = 4, TILE_BYTES = 9216;
    static constexpr bool SUMS = true;  // the matmul needs the activations' sub-block sums
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
    // the same tile copied byte for byte into LDS by the memory pipeline (no registers involved);
    // completion is counted by vmcnt like any other load
    static __device__ __forceinline__ void load_to_lds(uint32_t lds, const uint8_t* tile, int lane) {
#pragma unroll
        for (int u = 0; u < 9; u++) dma_to_lds_b128(tile + u * 1024 + lane * 16, lds + u * 1024);
    }
    // float index of this lane's sub-block sums of chunk c, before the row's own offset
    // (ActLoader::sumoff) is added: lane (b, i) reads sub-block b
    static __device__ __forceinline__ int xs_base(int c, int lane) { return c * 128 + ((lane >> 2) & 7) * 4; }
};

// Q5_K (crates/compute/src/quant_gguf/q5_k.rs:47-96): the Q4_K tile followed by the fifth bits,
// [2 units][64 lanes][16 B] = the lane's 32 qh bytes.
struct Q5K {
    static constexpr int NSUB = 8, NPAIR = 4, TILE_BYTES = 11264;
    static constexpr bool SUMS = true;
    struct Regs {
        u32x4 q[8];
        u32x4 s;
        u32x4 h[2];
    };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* tile, int lane) {
        const u32x4* p = (const u32x4*)tile + lane;
#pragma unroll
        for (int u = 0; u < 8; u++) r.q[u] = __builtin_nontemporal_load(p + u * 64);
        r.s = __builtin_nontemporal_load(p + 512);
        r.h[0] = __builtin_nontemporal_load(p + 576);
        r.h[1] = __builtin_nontemporal_load(p + 640);
    }
    static __device__ __forceinline__ int xs_base(int c, int lane) { return c * 128 + ((lane >> 2) & 7) * 4; }
};

struct Q80 {
    static constexpr int NSUB = 4, NPAIR = 2, TILE_BYTES = 8704;
    static constexpr bool SUMS = true;
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
    static __device__ __forceinline__ void load_to_lds(uint32_t lds, const uint8_t* tile, int lane) {
#pragma unroll
        for (int u = 0; u < 8; u++) dma_to_lds_b128(tile + u * 1024 + lane * 16, lds + u * 1024);
        // the 512-byte scale block: 8 bytes per lane, as two 4-byte transfers of 256 bytes
#pragma unroll
        for (int h = 0; h < 2; h++) dma_to_lds_b32(tile + 8192 + h * 256 + lane * 4, lds + 8192 + h * 256);
    }
    // a 128-element chunk is half of a 256-element sum group: its four sub-blocks go to blocks 0..3
    static __device__ __forceinline__ int xs_base(int c, int lane) {
        return (c >> 1) * 128 + (c & 1) * 16 + ((lane >> 2) & 3) * 4;
    }
};

// activation registers of one K chunk
// MXFP4 (ggml block_mxfp4: one e8m0 scale byte + 16 bytes of e2m1 nibbles per 32 elements;
// crates/compute/src/quant_gguf_mxfp4.rs:76-141).  A tile is 64 rows x 256 K: unit u holds the
// 32 nibbles of the lane's sub-block u, re-ordered at load time so that the four bytes of word w
// are K elements (8w, 8w+2), (8w+1, 8w+3), (8w+4, 8w+6), (8w+5, 8w+7) -- what
// v_cvt_scalef32_pk_f16_fp4 turns, byte by byte, into the fp16 pairs of two MFMA K steps in the
// activations' element order; then the eight scale bytes per lane.  e2m1 values are exact in
// fp16 and signed, so there is no code offset and no use for the activation sums.
struct MX4 {
    static constexpr int NSUB = 8, NPAIR = 4, TILE_BYTES = 8704;
    static constexpr bool SUMS = false;
    typedef Q80::Regs Regs;
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* tile, int lane) { Q80::load(r, tile, lane); }
    static __device__ __forceinline__ void load_to_lds(uint32_t lds, const uint8_t* tile, int lane) {
        Q80::load_to_lds(lds, tile, lane);
    }
    static __device__ __forceinline__ int xs_base(int c, int lane) { return Q4K::xs_base(c, lane); }
};

// bf16 matrices (crates/compute/src/quant.rs:14-39: a bf16 is the upper half of the fp32 bits).
// A tile is 64 rows x 64 K: unit u holds the lane's row at K steps 2u and 2u + 1, four values per
// step in the activations' element order (k % 4 = 0, 2, 1, 3), i.e. exactly the B operand of
// v_mfma_f32_4x4x4_16B_bf16.  The fp16 activations are split exactly into two bf16 terms
// (upper eight significant bits + remainder), so the products are those of the fp16 values.
struct BF16W {
    static constexpr int NSUB = 2, NPAIR = 1, TILE_BYTES = 8192;
    static constexpr bool SUMS = false;
    struct Regs {
        u32x4 q[8];
    };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* tile, int lane) {
        const u32x4* p = (const u32x4*)tile + lane;
#pragma unroll
        for (int u = 0; u < 8; u++) r.q[u] = __builtin_nontemporal_load(p + u * 64);
    }
    static __device__ __forceinline__ int xs_base(int, int) { return 0; }
};

// Q6_K (crates/compute/src/quant_gguf/q6_k.rs:44-88): value = d * sc_j * (level - 32), level = 4 low
// bits + 2 high bits, one signed int8 scale per 16 elements.  The level goes to the MFMA as the
// exact fp16 integer level - 32: (low nibble | 0x6400) | (high pair << 4) is 1024 + level, and one
// packed fp16 add of -1056 removes offset and bias together.
struct Q6K {
    static constexpr int NSUB = 16, NPAIR = 4, TILE_BYTES = 13568;
    static constexpr bool SUMS = false;
    struct Regs {
        u32x4 q[12];
        u32x4 s;
        uint32_t d;
    };
    static __device__ __forceinline__ void load(Regs& r, const uint8_t* tile, int lane) {
        const u32x4* p = (const u32x4*)tile + lane;
#pragma unroll
        for (int u = 0; u < 12; u++) r.q[u] = __builtin_nontemporal_load(p + u * 64);
        r.s = __builtin_nontemporal_load(p + 12 * 64);
        r.d = __builtin_nontemporal_load((const uint32_t*)(tile + 13312) + lane);
    }
    static __device__ __forceinline__ int xs_base(int, int) { return 0; }
};

template <int STEP>
__device__ __forceinline__ float4v mfma_bf16(u32x2 a, u32x2 b, float4v c) {
    typedef short short4v __attribute__((ext_vector_type(4)));
    return __builtin_amdgcn_mfma_f32_4x4x4bf16_1k(__builtin_bit_cast(short4v, a), __builtin_bit_cast(short4v, b), c, 4,
                                                  STEP, 0);
}

template <class F, int NG>
struct XRegs {
    u32x2 xa[F::NPAIR][NG];
    float xs[NG];
};

template <class F, int NG>
struct Stage {
    typename F::Regs w;
    XRegs<F, NG> x;
};

// Where a tile's bytes are read from while it is being multiplied: the registers of a stage, or
// the LDS copy made by load_to_lds (16 bytes per lane and unit, read just before use).
template <class F>
struct RegSrc {
    const typename F::Regs& r;
    __device__ __forceinline__ u32x4 unit(int u) const { return r.q[u]; }
    __device__ __forceinline__ auto scales() const { return r.s; }
    __device__ __forceinline__ auto dval() const { return r.d; }
    __device__ __forceinline__ u32x4 high(int u) const { return r.h[u]; }
};
template <class F>
struct LdsSrc {
    uint32_t base;  // LDS address (see lds_after)
    int lane;
    typedef decltype(typename F::Regs{}.s) Scales;
    __device__ __forceinline__ u32x4 unit(int u) const {
        return *(__attribute__((address_space(3))) const u32x4*)(uintptr_t)(base + (u * 64 + lane) * 16);
    }
    __device__ __forceinline__ Scales scales() const {
        return *(__attribute__((address_space(3))) const Scales*)(uintptr_t)(base + 8192 + lane * sizeof(Scales));
    }
};

// Cache policy of the activation loads: plain, or device-coherent (sc1) for activations that
// another compute unit wrote earlier in the same kernel (they must not come from this CU's L1).
// Which activation row feeds slot (g, i) of the MFMA A operand is a per-lane offset table: the
// identity for a dense matmul, a gather for a routed expert that sees only its own rows.
template <bool COHERENT>
struct ActLoader {
    __amdgpu_buffer_rsrc_t frag, sums;
    const u32x2* fragp;
    const float* sump;
    int rowoff[4], sumoff[4];  // offsets of row group g's row for this lane, in 8-byte units / floats
    __device__ __forceinline__ void set_row(int g, int row) {
        rowoff[g] = (row >> 2) * 64 + (row & 3);
        sumoff[g] = (row >> 2) * 32 + (row & 3);
    }
    // row `row` of a buffer made of 16-row blocks `block_bytes` apart (fragments and sums move together)
    __device__ __forceinline__ void set_row_blocked(int g, int row, size_t block_bytes) {
        set_row(g, row & 15);
        rowoff[g] += (int)((row >> 4) * (block_bytes >> 3));
        sumoff[g] += (int)((row >> 4) * (block_bytes >> 2));
    }
    __device__ __forceinline__ ActLoader(const void* xfrag, const void* xsum, int lane) {
        fragp = (const u32x2*)xfrag;
        sump = (const float*)xsum;
#pragma unroll
        for (int g = 0; g < 4; g++) set_row(g, 4 * g + (lane & 3));
        if (COHERENT) {
            frag = __builtin_amdgcn_make_buffer_rsrc((void*)xfrag, 0, 0x7FFFFFFF, 0x00027000);
            sums = __builtin_amdgcn_make_buffer_rsrc((void*)xsum, 0, 0x7FFFFFFF, 0x00027000);
        }
    }
    __device__ __forceinline__ u32x2 frag_at(int idx) const {  // idx in 8-byte units
        if (COHERENT) return __builtin_amdgcn_raw_buffer_load_b64(frag, idx * 8, 0, 16);
        return fragp[idx];
    }
    __device__ __forceinline__ float sum_at(int idx) const {
        if (COHERENT) return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(sums, idx * 4, 0, 16));
        return sump[idx];
    }
};

// activations of K chunk c (chunk index in the activation's own K axis)
template <class F, int NG, bool COH>
__device__ __forceinline__ void load_x(XRegs<F, NG>& xr, const ActLoader<COH>& x, int c, int lane) {
#pragma unroll
    for (int p = 0; p < F::NPAIR; p++)
#pragma unroll
        for (int g = 0; g < NG; g++) xr.xa[p][g] = x.frag_at((c * F::NPAIR + p) * 256 + x.rowoff[g] + (lane >> 2) * 4);
    if (F::SUMS) {
#pragma unroll
        for (int g = 0; g < NG; g++) xr.xs[g] = x.sum_at(F::xs_base(c, lane) + x.sumoff[g]);
    }
}

// The loads of one stage stay together and in program order (scheduling fences on both sides),
// so "stage s has landed" is one s_waitcnt vmcnt(n) with the same n on every path.
template <class F, int NG, bool COH>
__device__ __forceinline__ void load_stage(Stage<F, NG>& st, const ActLoader<COH>& x, const uint8_t* tile_chunk, int c,
                                           int lane) {
    __builtin_amdgcn_sched_barrier(0);
    load_x(st.x, x, c, lane);
    F::load(st.w, tile_chunk, lane);
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
template <int NG, class Src>
__device__ __forceinline__ void compute_tile(Q4K, const Src& w, const XRegs<Q4K, NG>& x, const Consts& k,
                                             float4v (&acc)[NG]) {
    const u32x4 hs = w.scales();
    const float d = h2f_lo(hs.x), dmin = h2f_hi(hs.x);
    // 6-bit scale / min unpack (q4_k.rs:43-54), four sub-blocks per 32-bit word
    const uint32_t sl = hs.y & 0x3F3F3F3Fu, ml = hs.z & 0x3F3F3F3Fu;
    const uint32_t sh = (hs.w & 0x0F0F0F0Fu) | ((hs.y >> 2) & 0x30303030u);
    const uint32_t mh = ((hs.w >> 4) & 0x0F0F0F0Fu) | ((hs.z >> 2) & 0x30303030u);
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
        for (int g = 0; g < NG; g++) t[g] = mfma_f32<j>(x.xs[g], cf[j], t[g]);
    });
#pragma unroll
    for (int p = 0; p < 4; p++) {
        const u32x4 qa = w.unit(2 * p), qb = w.unit(2 * p + 1);
        float4v dlo[NG], dhi[NG];
#pragma unroll
        for (int g = 0; g < NG; g++) dlo[g] = dhi[g] = float4v{0.f, 0.f, 0.f, 0.f};
        static_for<8>([&](auto W) {
            constexpr int wi = decltype(W)::value;
            const uint32_t word = wi < 4 ? qa[wi % 4] : qb[wi % 4];
            const uint32_t v = word >> 8;
            const u32x2 blo = {and_or(word, 0x000F000Fu, k.k6400), and_or(v, 0x000F000Fu, k.k6400)};
            const u32x2 bhi = {and_or(word, 0x00F000F0u, k.k5400), and_or(v, 0x00F000F0u, k.k5400)};
#pragma unroll
            for (int g = 0; g < NG; g++) {
                dlo[g] = mfma_f16<wi>(x.xa[p][g], blo, dlo[g]);
                dhi[g] = mfma_f16<wi + 8>(x.xa[p][g], bhi, dhi[g]);
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

// One Q5_K superblock tile: Q4_K's sequence with the fifth bit of every code OR-ed into the fp16
// integer before the MFMA (bit 4 of 1024 + q for the low-nibble elements, bit 8 of the 1/16-ulp
// 64 + q form for the high-nibble ones).  Byte l of the lane's 32 qh bytes serves elements l of all
// eight sub-blocks: sub-block pair p reads bit 2p (low nibbles) and bit 2p + 1 (high nibbles).
template <int NG, class Src>
__device__ __forceinline__ void compute_tile(Q5K, const Src& w, const XRegs<Q5K, NG>& x, const Consts& k,
                                             float4v (&acc)[NG]) {
    const u32x4 hs = w.scales();
    const float d = h2f_lo(hs.x), dmin = h2f_hi(hs.x);
    const uint32_t sl = hs.y & 0x3F3F3F3Fu, ml = hs.z & 0x3F3F3F3Fu;
    const uint32_t sh = (hs.w & 0x0F0F0F0Fu) | ((hs.y >> 2) & 0x30303030u);
    const uint32_t mh = ((hs.w >> 4) & 0x0F0F0F0Fu) | ((hs.z >> 2) & 0x30303030u);
    float sc[8], cf[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        sc[j] = d * ubyte(j < 4 ? sl : sh, j & 3);
        const float mn = dmin * ubyte(j < 4 ? ml : mh, j & 3);
        cf[j] = -__builtin_fmaf(sc[j], (j & 1) ? 64.0f : 1024.0f, mn);
    }
    float4v t[NG];
#pragma unroll
    for (int g = 0; g < NG; g++) t[g] = float4v{0.f, 0.f, 0.f, 0.f};
    static_for<8>([&](auto J) {
        constexpr int j = decltype(J)::value;
#pragma unroll
        for (int g = 0; g < NG; g++) t[g] = mfma_f32<j>(x.xs[g], cf[j], t[g]);
    });
    const u32x4 h0 = w.high(0), h1 = w.high(1);
    static_for<4>([&](auto P) {
        constexpr int p = decltype(P)::value;
        const u32x4 qa = w.unit(2 * p), qb = w.unit(2 * p + 1);
        float4v dlo[NG], dhi[NG];
#pragma unroll
        for (int g = 0; g < NG; g++) dlo[g] = dhi[g] = float4v{0.f, 0.f, 0.f, 0.f};
        static_for<8>([&](auto W) {
            constexpr int wi = decltype(W)::value;
            const uint32_t word = wi < 4 ? qa[wi % 4] : qb[wi % 4];
            const uint32_t hw = wi < 4 ? h0[wi % 4] : h1[wi % 4];
            const uint32_t v = word >> 8, hv = hw >> 8;
            // bit 2p of a qh byte -> bit 4 of its fp16 half; bit 2p + 1 -> bit 8
            constexpr int slo = 4 - 2 * p, shi = 7 - 2 * p;
            const uint32_t l0 = slo >= 0 ? hw << (slo >= 0 ? slo : 0) : hw >> (slo < 0 ? -slo : 0);
            const uint32_t l1 = slo >= 0 ? hv << (slo >= 0 ? slo : 0) : hv >> (slo < 0 ? -slo : 0);
            const uint32_t u0 = hw << shi, u1 = hv << shi;
            const u32x2 blo = {and_or(l0, 0x00100010u, and_or(word, 0x000F000Fu, k.k6400)),
                               and_or(l1, 0x00100010u, and_or(v, 0x000F000Fu, k.k6400))};
            const u32x2 bhi = {and_or(u0, 0x01000100u, and_or(word, 0x00F000F0u, k.k5400)),
                               and_or(u1, 0x01000100u, and_or(v, 0x00F000F0u, k.k5400))};
#pragma unroll
            for (int g = 0; g < NG; g++) {
                dlo[g] = mfma_f16<wi>(x.xa[p][g], blo, dlo[g]);
                dhi[g] = mfma_f16<wi + 8>(x.xa[p][g], bhi, dhi[g]);
            }
        });
#pragma unroll
        for (int g = 0; g < NG; g++) {
            fma4(t[g], sc[2 * p], dlo[g]);
            fma4(t[g], sc[2 * p + 1], dhi[g]);
        }
    });
#pragma unroll
    for (int g = 0; g < NG; g++) acc[g] += t[g];
}

// One Q8_0 tile (64 rows x 128 K = four 32-element blocks).  Codes go in as 1024 + (q + 128);
// the 1152 offset comes back out through the activation sums on the fp32 matrix pipe.
template <int NG, class Src>
__device__ __forceinline__ void compute_tile(Q80, const Src& w, const XRegs<Q80, NG>& x, const Consts& k,
                                             float4v (&acc)[NG]) {
    const u32x2 hs = w.scales();
    float dj[4] = {h2f_lo(hs.x), h2f_hi(hs.x), h2f_lo(hs.y), h2f_hi(hs.y)};
    float4v t[NG];
#pragma unroll
    for (int g = 0; g < NG; g++) t[g] = float4v{0.f, 0.f, 0.f, 0.f};
    static_for<4>([&](auto J) {
        constexpr int j = decltype(J)::value;
#pragma unroll
        for (int g = 0; g < NG; g++) t[g] = mfma_f32<j>(x.xs[g], dj[j] * -1152.0f, t[g]);
    });
#pragma unroll
    for (int p = 0; p < 2; p++) {
        const u32x4 qa0 = w.unit(4 * p), qa1 = w.unit(4 * p + 1), qb0 = w.unit(4 * p + 2), qb1 = w.unit(4 * p + 3);
        float4v da[NG], db[NG];
#pragma unroll
        for (int g = 0; g < NG; g++) da[g] = db[g] = float4v{0.f, 0.f, 0.f, 0.f};
        static_for<8>([&](auto W) {
            constexpr int wi = decltype(W)::value;
            // bytes -> fp16 1024 + (q + 128): interleave each byte with 0x64
            const uint32_t wa = (wi < 4 ? qa0[wi % 4] : qa1[wi % 4]) ^ 0x80808080u;
            const uint32_t wb = (wi < 4 ? qb0[wi % 4] : qb1[wi % 4]) ^ 0x80808080u;
            const u32x2 ba = {__builtin_amdgcn_perm(k.k64, wa, 0x04020400u), __builtin_amdgcn_perm(k.k64, wa, 0x04030401u)};
            const u32x2 bb = {__builtin_amdgcn_perm(k.k64, wb, 0x04020400u), __builtin_amdgcn_perm(k.k64, wb, 0x04030401u)};
#pragma unroll
            for (int g = 0; g < NG; g++) {
                da[g] = mfma_f16<wi>(x.xa[p][g], ba, da[g]);
                db[g] = mfma_f16<wi + 8>(x.xa[p][g], bb, db[g]);
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

// One MXFP4 tile (64 rows x 256 K = eight 32-element blocks): value = e2m1(code) * 2^(e - 127).
template <int NG, class Src>
__device__ __forceinline__ void compute_tile(MX4, const Src& w, const XRegs<MX4, NG>& x, const Consts&,
                                             float4v (&acc)[NG]) {
    typedef _Float16 half2v __attribute__((ext_vector_type(2)));
    const u32x2 hs = w.scales();
    float sc[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        const uint32_t e = ((j < 4 ? hs.x : hs.y) >> (8 * (j & 3))) & 0xFFu;
        sc[j] = __uint_as_float(e ? e << 23 : 0x00400000u);  // 2^(e-127); e = 0 is the subnormal 2^-127
    }
#pragma unroll
    for (int p = 0; p < 4; p++) {
        const u32x4 qa = w.unit(2 * p), qb = w.unit(2 * p + 1);
        float4v da[NG], db[NG];
#pragma unroll
        for (int g = 0; g < NG; g++) da[g] = db[g] = float4v{0.f, 0.f, 0.f, 0.f};
        static_for<4>([&](auto W) {
            constexpr int wi = decltype(W)::value;
            const uint32_t wa = qa[wi], wb = qb[wi];
            auto pair2 = [](uint32_t word, int lo) {
                const half2v h0 = lo ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, 1.0f, 2)
                                     : __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, 1.0f, 0);
                const half2v h1 = lo ? __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, 1.0f, 3)
                                     : __builtin_amdgcn_cvt_scalef32_pk_f16_fp4(word, 1.0f, 1);
                return u32x2{__builtin_bit_cast(uint32_t, h0), __builtin_bit_cast(uint32_t, h1)};
            };
            const u32x2 a0 = pair2(wa, 0), a1 = pair2(wa, 1), b0 = pair2(wb, 0), b1 = pair2(wb, 1);
#pragma unroll
            for (int g = 0; g < NG; g++) {
                da[g] = mfma_f16<2 * wi>(x.xa[p][g], a0, da[g]);
                da[g] = mfma_f16<2 * wi + 1>(x.xa[p][g], a1, da[g]);
                db[g] = mfma_f16<8 + 2 * wi>(x.xa[p][g], b0, db[g]);
                db[g] = mfma_f16<8 + 2 * wi + 1>(x.xa[p][g], b1, db[g]);
            }
        });
#pragma unroll
        for (int g = 0; g < NG; g++) {
            fma4(acc[g], sc[2 * p], da[g]);
            fma4(acc[g], sc[2 * p + 1], db[g]);
        }
    }
}

// One Q6_K superblock tile (64 rows x 256 K): sixteen 16-element sub-blocks, four K steps each.
template <int NG, class Src>
__device__ __forceinline__ void compute_tile(Q6K, const Src& w, const XRegs<Q6K, NG>& x, const Consts& k,
                                             float4v (&acc)[NG]) {
    typedef _Float16 half2v __attribute__((ext_vector_type(2)));
    const u32x4 scw = w.scales();
    const float d = h2f_lo(w.dval());
    const half2v off = {(_Float16)-1056.0f, (_Float16)-1056.0f};
#pragma unroll
    for (int p = 0; p < 4; p++) {
        const u32x4 n0 = w.unit(3 * p), n1 = w.unit(3 * p + 1), hh = w.unit(3 * p + 2);
        static_for<4>([&](auto Q) {
            constexpr int q = decltype(Q)::value;
            const uint32_t H = hh[q];
            float4v t[NG];
#pragma unroll
            for (int g = 0; g < NG; g++) t[g] = float4v{0.f, 0.f, 0.f, 0.f};
            static_for<4>([&](auto SI) {
                constexpr int si = decltype(SI)::value;
                constexpr int s = 4 * q + si;
                const uint32_t nw = s < 8 ? n0[(s & 7) >> 1] : n1[(s & 7) >> 1];
                auto build = [&](int ab) {
                    const int lo_sh = (s & 1) * 8 + 4 * ab, e = 2 * si + ab;
                    const uint32_t lo = and_or(nw >> lo_sh, 0x000F000Fu, k.k6400);
                    const uint32_t hi = 2 * e >= 4 ? H >> (2 * e - 4) : H << (4 - 2 * e);
                    const uint32_t v = and_or(hi, 0x00300030u, lo);  // 1024 + level, twice
                    return __builtin_bit_cast(uint32_t, __builtin_bit_cast(half2v, v) + off);
                };
                const u32x2 b = {build(0), build(1)};
#pragma unroll
                for (int g = 0; g < NG; g++) t[g] = mfma_f16<s>(x.xa[p][g], b, t[g]);
            });
            constexpr int j = 4 * q;  // sub-block 4p + q: byte (4p + q) of the scale unit
            const int sc8 = (int)(scw[p] << (24 - 8 * (j >> 2))) >> 24;
            const float sc = d * (float)sc8;
#pragma unroll
            for (int g = 0; g < NG; g++) fma4(acc[g], sc, t[g]);
        });
    }
}

// One bf16 tile (64 rows x 64 K).
template <int NG, class Src>
__device__ __forceinline__ void compute_tile(BF16W, const Src& w, const XRegs<BF16W, NG>& x, const Consts&,
                                             float4v (&acc)[NG]) {
    u32x2 ahi[NG], alo[NG];
#pragma unroll
    for (int g = 0; g < NG; g++) {
#pragma unroll
        for (int h = 0; h < 2; h++) {
            const uint32_t word = x.xa[0][g][h];
            const float f0 = h2f_lo(word), f1 = h2f_hi(word);
            const uint32_t b0 = __float_as_uint(f0) & 0xFFFF0000u, b1 = __float_as_uint(f1) & 0xFFFF0000u;
            const uint32_t r0 = __float_as_uint(f0 - __uint_as_float(b0)), r1 = __float_as_uint(f1 - __uint_as_float(b1));
            ahi[g][h] = (b0 >> 16) | b1;
            alo[g][h] = (r0 >> 16) | (r1 & 0xFFFF0000u);
        }
    }
    static_for<16>([&](auto S) {
        constexpr int s = decltype(S)::value;
        const u32x4 u = w.unit(s >> 1);
        const u32x2 b = (s & 1) ? u32x2{u.z, u.w} : u32x2{u.x, u.y};
#pragma unroll
        for (int g = 0; g < NG; g++) {
            acc[g] = mfma_bf16<s>(ahi[g], b, acc[g]);
            acc[g] = mfma_bf16<s>(alo[g], b, acc[g]);
        }
    });
}

// a register stage
template <class F, int NG>
__device__ __forceinline__ void compute(const Stage<F, NG>& st, const Consts& k, float4v (&acc)[NG]) {
    compute_tile<NG>(F{}, RegSrc<F>{st.w}, st.x, k, acc);
}

__device__ __forceinline__ float silu_f(float x) { return x / (1.0f + __expf(-x)); }

// The fused q/k/v projection finishing its own rows (no split-K: the sums are complete here).
// A tile of the rotated sections holds dims i (lanes 0..31) and i + hd/2 (lanes 32..63) of one
// head: the NeoX pair of a lane is lane ^ 32 (crates/compute/src/rope.rs:208-256).  Bias first,
// then the rotation (families/gptoss/attn.rs:88-118); q goes to the fp16 q buffer, K and V
// straight into the cache slot of the row (families/qwen/batched_layers.rs:84-113).
__device__ __forceinline__ void rope_epilogue(const RopeEpi& e, const VerifyParams* vp, int tile, int g, float4v v, int lane, int M) {
    const int hd = e.hd, half = hd >> 1, tph = hd >> 6;  // tiles per head
    const int tq = e.nq * tph, tk = e.nkv * tph;
    const int kind = tile < tq ? 0 : tile < tq + tk ? 1 : 2;
    const int st = kind == 0 ? tile : kind == 1 ? tile - tq : tile - tq - tk;
    const int head = st / tph, t = st - head * tph;
    const bool hi = lane >= 32;
    const int idim = (tph == 2 ? 32 * t : 0) + (lane & 31);     // rotation pair index, 0 .. hd/2
    const int d = kind == 2 ? t * 64 + lane : (hi ? idim + half : idim);  // this lane's head dimension
    const int col = (kind == 0 ? 0 : kind == 1 ? e.nq * hd : (e.nq + e.nkv) * hd) + head * hd + d;
    const float bias = e.bias ? e.bias[col] : 0.f;
    const int base = vp->base;
    float2 cs[4];
#pragma unroll
    for (int i = 0; i < 4; i++) cs[i] = kind != 2 && 4 * g + i < M ? e.cs[(4 * g + i) * half + idim] : float2{1.f, 0.f};
#pragma unroll
    for (int i = 0; i < 4; i++) {
        const int b = 4 * g + i;
        float x = v[i] + bias;
        const float other = __shfl_xor(x, 32);
        if (b >= M) continue;
        if (kind != 2) {
            const float x0 = hi ? other : x, x1 = hi ? x : other;
            x = hi ? x0 * cs[i].y + x1 * cs[i].x : x0 * cs[i].x - x1 * cs[i].y;
        }
        const _Float16 h = (_Float16)x;
        if (kind == 0) {
            ((_Float16*)e.q16)[((long)b * e.nq + head) * hd + d] = h;
        } else {
            const int pos = (base + b) % e.max_ctx;  // the cache slot of row b (a ring layer wraps at its capacity)
            if (kind == 1)
                ((_Float16*)e.kc)[kcache_index(head, pos, d, hd, e.max_ctx)] = h;
            else
                ((_Float16*)e.vc)[vcache_index(head, pos, d, hd, e.max_ctx)] = h;
        }
    }
}

}  // namespace tsv
