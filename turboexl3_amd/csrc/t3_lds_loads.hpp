// Loads that go from memory straight into LDS on gfx950 (buffer_load_dwordx4 ... lds), as the GEMV's and the GEMMs'
// operand rings use them. The instruction is issued from inline asm, so the compiler neither sees nor waits for these
// loads: a kernel that uses them counts them itself (wait_loads) and knows what else of its own is in the wave's queue
// of vector-memory operations (they complete in order: anything else in the queue only makes a wait longer, never
// shorter than it has to be).
#pragma once

#include "t3_common.hpp"

namespace t3 {

// A raw buffer descriptor as four scalars, and a wave's load of 16 bytes a lane from it straight into LDS: lane L's
// bytes land at lds + 16 L, from byte voff (the lane's) + soff (uniform) of the buffer; past the buffer's end they are
// zeros.
__device__ __forceinline__ uint4v rsrc_words(const void* p, uint64_t bytes) {
    const uint64_t addr = reinterpret_cast<uint64_t>(p);
    const uint32_t n = bytes > 0xFFFFFFFFull ? 0xFFFFFFFFu : static_cast<uint32_t>(bytes);
    return uint4v{static_cast<uint32_t>(addr), static_cast<uint32_t>(addr >> 32) & 0xFFFFu, n, 0x00020000u};
}
// (m0 is named as clobbered so the compiler keeps nothing of its own in it across the statement; clang warns about any
// reserved register in a clobber list, which is the point here)
#pragma clang diagnostic push
#pragma clang diagnostic ignored "-Winline-asm"
__device__ __forceinline__ void load_to_lds(uint4v desc, uint32_t lds, uint32_t voff, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds), "v"(voff), "s"(desc), "s"(soff)
                 : "memory", "m0");
}
#pragma clang diagnostic pop
// at most N of the wave's loads are still in flight (they complete in order)
template <int N>
__device__ __forceinline__ void wait_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}
// every LDS read the wave has issued has returned
__device__ __forceinline__ void wait_lds_reads() { asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory"); }

}  // namespace t3
