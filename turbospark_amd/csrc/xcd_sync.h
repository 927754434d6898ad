// XCD-local synchronisation for kernels that treat the eight XCDs of an MI355X like tensor-parallel
// devices: a workgroup finds out which XCD it runs on and its rank among that XCD's 32 workgroups,
// and the 32 meet at barriers kept in the XCD's own L2 (~0.7 us; a device-wide barrier costs about as
// much as ending the kernel).  Memory rules (measured on this part): plain stores followed by
// s_waitcnt vmcnt(0) and the XCD barrier are visible to sc1 ("device-coherent") loads from any
// compute unit of the same XCD; plain loads may hit a stale line in the reader's L1.
// Every wait is bounded: a barrier that does not complete within its spin budget raises the error
// flag and the workgroup returns, so the grid always drains.
#pragma once
#include "tsv_internal.h"

namespace tsv {
namespace {

constexpr int XCDS = 8;
constexpr int WGS_PER_XCD = 32;
constexpr unsigned SPIN_LIMIT = 1u << 21;

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

// Workgroup barrier that waits for LDS traffic only: global loads asked for earlier (weight
// prefetches) stay in flight across it.  (__syncthreads() carries a release fence that drains them.)
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// One 32-bit word read past the scalar cache.  A scalar load is counted by lgkmcnt, not vmcnt, so a
// wave with vector loads in flight can poll a flag without first waiting for all of them (vector
// loads return through one in-order counter: the answer to a vector poll could only be looked at
// after every older prefetch had landed).
__device__ __forceinline__ unsigned poll_u32(const unsigned* p) {
    const unsigned long long a = (unsigned long long)(uintptr_t)p;
    const unsigned lo = __builtin_amdgcn_readfirstlane((unsigned)a), hi = __builtin_amdgcn_readfirstlane((unsigned)(a >> 32));
    const unsigned long long ua = ((unsigned long long)hi << 32) | lo;
    unsigned v;
    asm volatile("s_load_dword %0, %1, 0x0 glc\n\ts_waitcnt lgkmcnt(0)" : "=s"(v) : "s"(ua) : "memory");
    return v;
}

// Barrier over the 32 workgroups of this XCD.  A wave that stored something the other side of
// the barrier will read first waits for its stores to be acknowledged by the L2 (drain); a wave
// that only has weight prefetches in flight must not wait for those here.
__device__ __forceinline__ bool xcd_barrier(XcdCtx& c, int* lds_i, bool drain = true) {
    if (drain) asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)" ::: "memory");
    lds_barrier();
    if (threadIdx.x == 0) {
        __hip_atomic_fetch_add(c.bar, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        unsigned n = 0;
        int ok = 1;
        while ((int)(poll_u32(c.bar) - c.next_target) < 0) {
            if (++n > SPIN_LIMIT) {
                ok = 0;
                *c.err = 1;
                break;
            }
            __builtin_amdgcn_s_sleep(1);
        }
        lds_i[2] = ok;
    }
    lds_barrier();
    c.next_target += WGS_PER_XCD;
    const bool ok = lds_i[2] != 0;
    lds_barrier();
    return ok;
}

__device__ __forceinline__ float ld_sc1(const float* base, int idx) {
    const __amdgpu_buffer_rsrc_t r = __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, 0x7FFFFFFF, 0x00027000);
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(r, idx * 4, 0, 16));
}

}  // namespace
}  // namespace tsv
