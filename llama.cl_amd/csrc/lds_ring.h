// Weight streaming through LDS: direct global->LDS loads into per-wave rings of step slots, the
// hand-placed waits that go with them, and the reads that turn a slot back into a Step<G>.
#pragma once
#include "common.h"
#include "gemv_device.h"

namespace llmops {

template <int G>
struct RingCfg {
    static constexpr int kStepBytes = Step<G>::kBlocksPerStep * (int)block_bytes(G);  // 2176 / 1280
    static constexpr int kLoads = (kStepBytes + 1023) / 1024;                         // wave-wide 16 B loads per step
};

// One 16-byte-per-lane asynchronous copy global -> LDS: lane i's 16 bytes land at lds_base + 16*i.
// Written as assembly on purpose.  The compiler, when it knows that such copies are pending, makes
// every later LDS access wait for all of them (it cannot tell which LDS bytes they target), which
// would serialise the ring; this way it sees an opaque memory operation, and the waits on the ring
// are placed by hand (wait_vm).  Hidden loads are harmless for the waits the compiler places for its
// own loads: loads complete in issue order, so an unknown older load only makes such a wait longer.
__device__ __forceinline__ void dma16(const uint8_t* gptr, uint32_t lds_base) {
    asm volatile(
        "s_mov_b32 m0, %1\n\t"
        "s_nop 0\n\t"
        "global_load_lds_dwordx4 %0, off nt"
        :
        : "v"(gptr), "s"(lds_base)
        : "memory", "m0");
}

__device__ __forceinline__ uint32_t lds_addr(const void* p) {
    return (uint32_t)(uintptr_t)((const __attribute__((address_space(3))) void*)p);
}

// one step of the weight stream, global -> LDS (counts in vmcnt)
template <int G>
__device__ __forceinline__ void ring_issue(const uint8_t* src, uint8_t* slot, int lane) {
    constexpr int SB = RingCfg<G>::kStepBytes;
    const uint32_t base = __builtin_amdgcn_readfirstlane(lds_addr(slot));
#pragma unroll
    for (int o = 0; o < SB; o += 1024) {
        if (SB - o >= 1024) {
            dma16(src + o + lane * 16, base + o);
        } else if (lane * 16 < SB - o) {
            dma16(src + o + lane * 16, base + o);
        }
    }
}

template <int G>
__device__ __forceinline__ void ring_read(Step<G>& st, const uint8_t* slot, int lane) {
    const int quad = lane & 7, rs = lane >> 3;
    st.valid = true;
    if (G == 128) {
        st.w[0] = *reinterpret_cast<const uint4*>(slot + lane * 16);
        st.w[Step<G>::kLoads - 1] = *reinterpret_cast<const uint4*>(slot + 1024 + lane * 16);
        st.dh = *reinterpret_cast<const uint2*>(slot + 2048 + quad * 8);
        st.mh = *reinterpret_cast<const uint2*>(slot + 2048 + 64 + quad * 8);
    } else {
        const uint8_t* blk = slot + (rs >> 2) * (int)block_bytes(32);
        st.w[0] = *reinterpret_cast<const uint4*>(blk + (rs & 3) * kRowBytes + quad * 16);
        st.dh = *reinterpret_cast<const uint2*>(blk + 512 + quad * 8);
        st.mh = *reinterpret_cast<const uint2*>(blk + 512 + 64 + quad * 8);
    }
}

// wait until at most `loads` of this wave's vector-memory operations are outstanding
__device__ __forceinline__ void wait_vm(int loads) {
    switch (loads) {
#define LLMOPS_W(n) \
    case n:         \
        asm volatile("s_waitcnt vmcnt(" #n ")" ::: "memory"); \
        break;
        LLMOPS_W(1) LLMOPS_W(2) LLMOPS_W(3) LLMOPS_W(4) LLMOPS_W(5) LLMOPS_W(6) LLMOPS_W(7) LLMOPS_W(8)
        LLMOPS_W(9) LLMOPS_W(10) LLMOPS_W(11) LLMOPS_W(12) LLMOPS_W(13) LLMOPS_W(14) LLMOPS_W(15) LLMOPS_W(16)
        LLMOPS_W(17) LLMOPS_W(18) LLMOPS_W(19) LLMOPS_W(20) LLMOPS_W(21) LLMOPS_W(22) LLMOPS_W(23) LLMOPS_W(24)
#undef LLMOPS_W
        default:
            asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
            break;
    }
}

}  // namespace llmops
