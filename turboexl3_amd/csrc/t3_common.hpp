// Shared device helpers of the gfx950 EXL3 kernels: dtypes, f16/bf16 conversions, the 128-point Hadamard of one
// wave64, and the constants of the format (turboexl3 src/core/format.zig:10-16).
#pragma once

#include <hip/hip_runtime.h>

#include <cstdint>

namespace t3 {

// Activation dtypes by the C ABI's t3_dtype numbers (T3_F32, T3_F16, T3_BF16), which are the reference plan's
// (turboexl3 src/hip/plan.zig:72-73): a launch descriptor carries the caller's number straight through.
enum Dtype : int { kF32, kF16, kBf16 };
static_assert(kF32 == 0 && kF16 == 1 && kBf16 == 2, "the ABI's dtype numbers");

constexpr int kWave = 64;
// a Hadamard-128 is orthonormal with this factor: 2^-3.5
constexpr float kHadScale = 0.088388347648318440550105545263106f;

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float float4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));
typedef uint32_t uint2v __attribute__((ext_vector_type(2)));

// A raw buffer over `bytes` bytes from p: loads take a per-lane byte offset (VGPR) plus a uniform byte offset (SGPR),
// so a streaming loop spends no vector ALU on addresses, and a read past the end returns zero instead of faulting.
__device__ __forceinline__ __amdgpu_buffer_rsrc_t make_rsrc(const void* p, uint64_t bytes) {
    const uint32_t n = bytes > 0xFFFFFFFFull ? 0xFFFFFFFFu : static_cast<uint32_t>(bytes);
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(p), 0, static_cast<int>(n), 0x00020000);
}
__device__ __forceinline__ uint32_t buf_load_u32(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    return __builtin_amdgcn_raw_buffer_load_b32(r, static_cast<int>(voff), static_cast<int>(soff), 0);
}
__device__ __forceinline__ uint4v buf_load_u128(__amdgpu_buffer_rsrc_t r, uint32_t voff, uint32_t soff) {
    return __builtin_amdgcn_raw_buffer_load_b128(r, static_cast<int>(voff), static_cast<int>(soff), 0);
}

// Device-coherent accesses for data that crosses workgroups inside one launch. The GPU's eight dies each have their
// own L2, so a device-scope fence writes back and invalidates a whole L2: ruinous when every workgroup runs one.
// Relaxed device-scope atomic loads and stores go to the coherent level by themselves (the sc1 cache policy) and leave
// every other access cached.
__device__ __forceinline__ void store_coherent(float* p, float v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
__device__ __forceinline__ float load_coherent(const float* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
// four adjacent floats (16-byte aligned) in one device-coherent store. The two wait states behind it: a store of more
// than 64 bits reads its data registers over several cycles, and a vector instruction that writes one of them right
// behind the store changes what the later lanes store. The compiler keeps that distance for its own stores; it does not
// look inside this one. (Seen once the register allocation put a v_mov into the store's first two data registers as
// the next instruction: lanes 12-15 and 28-31 of the wave stored the new values in their first two floats.)
__device__ __forceinline__ void store_coherent4(float* p, float4v v) {
    asm volatile("global_store_dwordx4 %0, %1, off sc1\n\ts_nop 1" : : "v"(p), "v"(v) : "memory");
}
// every store this lane has issued is acknowledged at its coherence level (with store_coherent: device-wide)
__device__ __forceinline__ void wait_stores() { asm volatile("s_waitcnt vmcnt(0)" ::: "memory"); }

// ---- activation elements ----------------------------------------------------------------------------------------
// f16 values travel as their 16-bit patterns where they are packed by hand (two to a register for the matrix core).
__device__ __forceinline__ float half_value(uint32_t bits) {
    return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(bits)));
}
__device__ __forceinline__ uint16_t half_bits(float v) {
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(v));
}
// v rounded to the nearest f16 and back: format.project's rounding points (turboexl3 src/core/format.zig:144-146)
__device__ __forceinline__ float round_half(float v) { return static_cast<float>(static_cast<_Float16>(v)); }

// bf16 is the top half of an f32. Narrowing is the hardware's (gfx950 converts f32 -> bf16 to nearest even in one
// instruction, v_cvt_pk_bf16_f32, which is what the cast below compiles to); a NaN is kept apart so that it leaves with
// its own sign and top payload bits and the quiet bit set, the host-side rule the outputs are checked against
// (turboexl3 src/test_support.zig:14-19).
typedef __bf16 bf16_t;
__device__ __forceinline__ float bf16_value(uint16_t b) {
    return static_cast<float>(__builtin_bit_cast(bf16_t, b));
}
__device__ __forceinline__ uint16_t bf16_bits(float v) {
    const uint16_t nearest = __builtin_bit_cast(uint16_t, static_cast<bf16_t>(v));
    const uint16_t quiet = static_cast<uint16_t>(__builtin_bit_cast(uint32_t, v) >> 16) | 0x40u;
    return v != v ? quiet : nearest;
}

// How an activation dtype sits in memory and crosses to f32: one description a dtype, used by every typed load and
// store of the kernels (a store rounds once, to nearest even).
template <int DT>
struct ActElem;
template <>
struct ActElem<kF32> {
    typedef float Stored;
    static __device__ __forceinline__ float widen(Stored s) { return s; }
    static __device__ __forceinline__ Stored narrow(float v) { return v; }
};
template <>
struct ActElem<kF16> {
    typedef _Float16 Stored;
    static __device__ __forceinline__ float widen(Stored s) { return static_cast<float>(s); }
    static __device__ __forceinline__ Stored narrow(float v) { return static_cast<Stored>(v); }
};
template <>
struct ActElem<kBf16> {
    typedef uint16_t Stored;
    static __device__ __forceinline__ float widen(Stored s) { return bf16_value(s); }
    static __device__ __forceinline__ Stored narrow(float v) { return bf16_bits(v); }
};
template <int DT>
__device__ __forceinline__ float load_act(const void* base, size_t index) {
    return ActElem<DT>::widen(static_cast<const typename ActElem<DT>::Stored*>(base)[index]);
}
template <int DT>
__device__ __forceinline__ void store_act(void* base, size_t index, float v) {
    static_cast<typename ActElem<DT>::Stored*>(base)[index] = ActElem<DT>::narrow(v);
}

// The unscaled Hadamard of a 128-block held by one wave64: lane L owns elements L and L + 64 (v[0], v[1]).
// Six cross-lane stages over element bits 0..5, then the lane's own stage over bit 6. The stage order is fixed: every
// kernel that transforms a block uses this function, so a block's bits do not depend on which kernel transformed it.
__device__ __forceinline__ void h128_wave(float (&v)[2], uint32_t lane) {
#pragma unroll
    for (uint32_t s = 0; s < 6u; ++s) {
        const uint32_t bit = 1u << s;
#pragma unroll
        for (uint32_t j = 0; j < 2u; ++j) {
            const float p = __shfl_xor(v[j], static_cast<int>(bit), 64);
            v[j] = (lane & bit) ? (p - v[j]) : (v[j] + p);
        }
    }
    const float a = v[0] + v[1], b = v[0] - v[1];
    v[0] = a;
    v[1] = b;
}

// Slot of element r (0..15) of a 16-input tile in "quad order": the four inputs a lane's weights multiply,
// tile rows 2q + {0, 1, 8, 9}, sit at slots 4q..4q+3 (turboexl3 src/kernels/hip/common.hpp:70-75 uses the same order).
__device__ __forceinline__ uint32_t quad_slot(uint32_t r) {
    const uint32_t q = (r & 7u) >> 1u;
    const uint32_t m = (r & 1u) | ((r >> 3u) << 1u);
    return 4u * q + m;
}

// Where input i of a row sits in the prepared activations the GEMM reads ("pair-quad order"): inside every 32 inputs
// (two tile rows A, B), quad q of A then quad q of B, q = 0..3: the 16 bytes at q are the eight K slots of the MFMA's B
// fragment that meet a lane's eight weights (tile rows 2q + {0, 1, 8, 9} of A, then of B).
__device__ __forceinline__ uint32_t pair_quad_slot(uint32_t i) {
    const uint32_t r = i & 15u;
    const uint32_t q = (r & 7u) >> 1u, m = (r & 1u) | ((r >> 3u) << 1u);
    return (i & ~31u) + 8u * q + 4u * ((i >> 4u) & 1u) + m;
}

// Where arrival counter i of a launch's `count` counters sits in the workspace's head (16,384 words): a cache line apart
// while they fit (32 words), else 8 words, else side by side. A launch's workgroups count themselves in within a
// microsecond of one another, and atomics to one cache line queue up: sixteen counters to a line cost the routed decode's
// down launch, 176 arrivals at one token, a microsecond.
__device__ __forceinline__ uint32_t arrive_slot(uint32_t i, uint32_t count) {
    return i * (count <= 512u ? 32u : (count <= 2048u ? 8u : 1u));
}

// MUL1's affine map w = A h + B with h = 1024 + t (format.zig:158-167): A = f16 0x1EEE, B = f16 0xC931
__device__ __forceinline__ float mul1_a() { return half_value(0x1EEEu); }
__device__ __forceinline__ float mul1_b() { return half_value(0xC931u); }

}  // namespace t3
