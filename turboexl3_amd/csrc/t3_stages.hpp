// The per-block arithmetic of a projection's prepare and finish, shared by the dense and the routed kernels: one
// wave64 a 128-block, lane L owning elements L and L + 64 (format.project's stages, turboexl3
// src/core/format.zig:334-380, with its rounding points).
#pragma once

#include "t3_common.hpp"

namespace t3 {

__device__ __forceinline__ float load_act_rt(int dt, const void* p, size_t i) {
    if (dt == kF32) return load_act<kF32>(p, i);
    if (dt == kF16) return load_act<kF16>(p, i);
    return load_act<kBf16>(p, i);
}
__device__ __forceinline__ void store_act_rt(int dt, void* p, size_t i, float v) {
    if (dt == kF32) store_act<kF32>(p, i, v);
    else if (dt == kF16) store_act<kF16>(p, i, v);
    else store_act<kBf16>(p, i, v);
}

// The prepare of one 128-block from its scaled inputs v = f16(x) * suh (lane L owns elements L and L + 64): the
// lane's two prepared f16 values (bits) and the block's sum of them (the same in every lane).
// want_sum false (uniform): the sum is not needed (only MUL1's deferred map reads it) and comes back 0.
__device__ __forceinline__ void prep_core(float (&v)[2], uint32_t lane, uint32_t (&hv)[2], float& sum,
                                          bool want_sum = true) {
    h128_wave(v, lane);
    sum = 0.0f;
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
        hv[j] = half_bits(v[j] * kHadScale);
        sum += half_value(hv[j]);
    }
    if (!want_sum) {
        sum = 0.0f;
        return;
    }
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) sum += __shfl_xor(sum, m, 64);
}

// One 128-block of one row, one wave: loads, then prep_core.
__device__ __forceinline__ void prep_values(int dt, const void* x, const uint16_t* suh, uint32_t in, uint32_t row,
                                            uint32_t b, uint32_t lane, uint32_t (&hv)[2], float& sum) {
    float v[2];
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
        const uint32_t i = b * 128u + lane + 64u * j;
        v[j] = round_half(load_act_rt(dt, x, static_cast<size_t>(row) * in + i)) * half_value(suh[i]);
    }
    prep_core(v, lane, hv, sum);
}

// The block's outputs from its summed inner products: f16, H128, * svh / sqrt(128), f16. s[j]: the lane's two sums
// (already through the deferred map when there is one); sv: the lane's two svh values; returns the two finished values
// (f16-valued).
__device__ __forceinline__ void finish_core(float (&s)[2], const float (&sv)[2], uint32_t lane) {
    float v[2] = {round_half(s[0]), round_half(s[1])};
    h128_wave(v, lane);
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) s[j] = round_half(v[j] * kHadScale * sv[j]);
}
__device__ __forceinline__ void finish_values(float (&s)[2], const uint16_t* svh, uint32_t b, uint32_t lane) {
    const float sv[2] = {half_value(svh[b * 128u + lane]), half_value(svh[b * 128u + lane + 64u])};
    finish_core(s, sv, lane);
}

// One element's SwiGLU in f32 on the f16-valued gate and up, with the clamp (turboexl3 src/core/ref.zig:119-140): limit 0
// none; clamp_at 0 (gate_in) silu(min(g, L)) * clamp(u, -L, L); clamp_at 1 (silu_out) min(silu(g), L) * clamp(u, -L, L).
// Comparisons, so a NaN passes through.
__device__ __forceinline__ float swiglu_clamped(float g, float u, float limit, int clamp_at) {
    if (limit > 0.0f) {
        u = u > limit ? limit : (u < -limit ? -limit : u);
        if (clamp_at == 0) g = g > limit ? limit : g;
    }
    float sg = g / (1.0f + expf(-g));
    if (limit > 0.0f && clamp_at != 0) sg = sg > limit ? limit : sg;
    return sg * u;
}

}  // namespace t3
