// Hand-over between two kernels of a pass that run on different streams at the same time: the
// consumer is started early, asks for everything that does not depend on the producer (its first
// weight tiles, old cache rows) and then waits here for the producer's last workgroup.  There is
// no kernel boundary between the two, hence no cache write-back / invalidate either: what the
// producer hands over it stores device-coherently (sc1: written through to memory), and the
// consumer reads it device-coherently (sc1: past its own die's L2).
//
// A slot is 81 words, each on a cache line of its own: sixteen group counters, one top counter,
// sixty-four copies of the "ready" word.  A producer workgroup, once all its stores are
// acknowledged, counts itself into group (index % 16); the last of a group counts the group into
// the top counter; the last group clears the counters and writes the launch's epoch to all copies
// of the ready word.  Two levels because atomics on one line are served one after the other
// (about 10 ns each: 448 workgroups arriving together on one counter wait 4.5 us); sixty-four
// copies because polls of one line are served one after the other as well (a consumer workgroup
// polls copy index % 64).  Epochs only grow (compared wrap-safe), so the ready words are never
// reset; the host hands every producer launch of a slot the next epoch.
// Every wait is bounded: a poll that runs out raises the error word and the kernel goes on and
// exits normally (its results are then garbage and the host reports the pass as failed).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace tsv {

constexpr int HANDOFF_LINE = 32;                // words between two of a slot's words (128 bytes)
constexpr int HANDOFF_GROUPS = 16;
constexpr int HANDOFF_COPIES = 64;
constexpr int HANDOFF_SLOT_WORDS = (HANDOFF_GROUPS + 1 + HANDOFF_COPIES) * HANDOFF_LINE;
constexpr unsigned HANDOFF_SPIN_LIMIT = 1u << 17;  // polls of about half a microsecond each

struct Handoff {
    const unsigned* wait;  // nullable: the slot this launch waits on
    unsigned* sig;         // nullable: the slot this launch signals
    unsigned wait_epoch, sig_epoch;
    int* err;              // set to 1 when a wait ran out
};

// device-coherent accesses (sc1) through the buffer instructions, so that several can be in flight
// (an atomic load is followed by a full wait) and 16-bit values can be stored
__device__ __forceinline__ __amdgpu_buffer_rsrc_t coh_rsrc(const void* base) {
    return __builtin_amdgcn_make_buffer_rsrc((void*)base, 0, 0x7FFFFFFF, 0x00027000);
}
constexpr int COH_AUX = 16;  // sc1
__device__ __forceinline__ void coh_store_f32(float* p, float v) {
    __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(uint32_t, v), coh_rsrc(p), 0, 0, COH_AUX);
}
__device__ __forceinline__ void coh_store_u32(uint32_t* p, uint32_t v) {
    __builtin_amdgcn_raw_buffer_store_b32(v, coh_rsrc(p), 0, 0, COH_AUX);
}
__device__ __forceinline__ void coh_store_f16(_Float16* p, _Float16 v) {
    __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(uint16_t, v), coh_rsrc(p), 0, 0, COH_AUX);
}
__device__ __forceinline__ float coh_load_f32(const float* p) {
    return __builtin_bit_cast(float, __builtin_amdgcn_raw_buffer_load_b32(coh_rsrc(p), 0, 0, COH_AUX));
}

__device__ __forceinline__ int handoff_block_index() {
    return (int)(blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z));
}
__device__ __forceinline__ int handoff_block_count() { return (int)(gridDim.x * gridDim.y * gridDim.z); }

// Consumer: returns once the producer of h.wait has published h.wait_epoch (or the poll ran out).
// Called by every wave of the workgroup, in uniform control flow.  Loads asked for before the call
// stay in flight across it (the barrier waits for LDS traffic only).
__device__ __forceinline__ void handoff_wait(const Handoff& h) {
    if (!h.wait) return;
    if (threadIdx.x < 64) {
        const unsigned* p = h.wait + (HANDOFF_GROUPS + 1 + (handoff_block_index() & (HANDOFF_COPIES - 1))) * HANDOFF_LINE;
        unsigned n = 0;
        while ((int)(__hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) - h.wait_epoch) < 0) {
            if (++n > HANDOFF_SPIN_LIMIT) {
                if (threadIdx.x == 0) __hip_atomic_store(h.err, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                break;
            }
            __builtin_amdgcn_s_sleep(8);
        }
    }
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Producer: called by every wave of the workgroup, in uniform control flow, after its last store.
__device__ __forceinline__ void handoff_signal(const Handoff& h) {
    if (!h.sig) return;
    asm volatile("s_waitcnt vmcnt(0) lgkmcnt(0)\n\ts_barrier" ::: "memory");  // every wave's stores are acknowledged
    if (threadIdx.x >= 64) return;
    const int lane = threadIdx.x;
    unsigned last = 0;
    if (lane == 0) {
        const int idx = handoff_block_index(), n = handoff_block_count();
        const int g = idx & (HANDOFF_GROUPS - 1);
        const unsigned in_group = (unsigned)(n - g + HANDOFF_GROUPS - 1) / HANDOFF_GROUPS;
        const unsigned groups = n < HANDOFF_GROUPS ? (unsigned)n : (unsigned)HANDOFF_GROUPS;
        if (__hip_atomic_fetch_add(h.sig + g * HANDOFF_LINE, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 == in_group)
            if (__hip_atomic_fetch_add(h.sig + HANDOFF_GROUPS * HANDOFF_LINE, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 == groups)
                last = 1;
    }
    if (!__builtin_amdgcn_readfirstlane(last)) return;
    if (lane <= HANDOFF_GROUPS) __hip_atomic_store(h.sig + lane * HANDOFF_LINE, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store(h.sig + (HANDOFF_GROUPS + 1 + lane) * HANDOFF_LINE, h.sig_epoch, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

}  // namespace tsv
