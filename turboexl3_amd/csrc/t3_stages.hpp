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
// round_x false: GLM's profile, x times suh in f32 without the f16 rounding of x.
__device__ __forceinline__ void prep_values(int dt, const void* x, const uint16_t* suh, uint32_t in, uint32_t row,
                                            uint32_t b, uint32_t lane, uint32_t (&hv)[2], float& sum,
                                            bool round_x = true) {
    float v[2];
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
        const uint32_t i = b * 128u + lane + 64u * j;
        const float xr = load_act_rt(dt, x, static_cast<size_t>(row) * in + i);
        v[j] = (round_x ? round_half(xr) : xr) * half_value(suh[i]);
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

// GLM's rounding profile (turboexl3 src/kernels/hip/decode/decode.hip:8-13, routed.hpp:89-98,120-133): the inner
// products stay f32 (no f16 rounding before a finish); gate and up round to bf16 and are limited, the SiLU rounds to
// bf16, the product rounds to bf16; a down finish stays f32.
__device__ __forceinline__ float round_bf16(float v) { return bf16_value(bf16_bits(v)); }
__device__ __forceinline__ void finish_core_glm(float (&s)[2], const float (&sv)[2], uint32_t lane, bool to_bf16) {
    h128_wave(s, lane);
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
        s[j] = s[j] * kHadScale * sv[j];
        if (to_bf16) s[j] = round_bf16(s[j]);
    }
}
// g, u: bf16 values. limit 0: none; a NaN stays a NaN (torch.clamp).
__device__ __forceinline__ float swiglu_glm(float g, float u, float limit) {
    if (limit > 0.0f) {
        g = g > limit ? limit : g;
        u = u > limit ? limit : (u < -limit ? -limit : u);
    }
    return round_bf16(round_bf16(g / (1.0f + expf(-g))) * u);
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

// ---- the same stages, four 128-blocks a wave --------------------------------------------------------------------
// 16 lanes a block, 8 adjacent elements a lane: element 8 q + r of the block, q = lane % 16. The butterflies are
// h128_wave's, in its order (element bits 0..6), so a block's bits do not depend on the layout that transformed it.
// Bits 0..2 pair registers. Bits 3..6 pair lanes q ^ 1, 2, 4, 8 through DPP; there the lane keeps t with value = S t,
// S = the product of the passed stages' signs (s = -1 on the lanes whose bit is set): partner lanes share S, and
// (bit set ? p - v : v + p) = s (t + s t_p), so a stage is one multiply-add a value and S leaves with the final scale.

struct Row16 {
    float s1, s2, s4, s8;  // the four lane stages' signs
    float scale;           // their product / sqrt(128)
};
__device__ __forceinline__ Row16 row16(uint32_t lane) {
    Row16 g;
    g.s1 = (lane & 1u) ? -1.0f : 1.0f;
    g.s2 = (lane & 2u) ? -1.0f : 1.0f;
    g.s4 = (lane & 4u) ? -1.0f : 1.0f;
    g.s8 = (lane & 8u) ? -1.0f : 1.0f;
    g.scale = g.s1 * g.s2 * g.s4 * g.s8 * kHadScale;
    return g;
}

// v of another lane of the row of 16 (CTRL: the DPP control). dpp_fill: the same for the lanes of BANK (a mask over
// the row's groups of 4 lanes), the others keep old.
template <int CTRL>
__device__ __forceinline__ float dpp_take(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_mov_dpp(__builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
template <int CTRL, int BANK>
__device__ __forceinline__ float dpp_fill(float old, float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(__builtin_bit_cast(int, old), __builtin_bit_cast(int, v),
                                                                 CTRL, 0xF, BANK, false));
}
constexpr int kDppXor1 = 0xB1, kDppXor2 = 0x4E;         // quad_perm [1,0,3,2], [2,3,0,1]
constexpr int kDppRor4 = 0x124, kDppRor8 = 0x128, kDppRor12 = 0x12C;  // lane i reads lane (i - n) mod 16

__device__ __forceinline__ void h128_row16(float (&v)[8], const Row16& g) {
#pragma unroll
    for (uint32_t bit = 1; bit < 8u; bit <<= 1)
#pragma unroll
        for (uint32_t r = 0; r < 8u; ++r)
            if (!(r & bit)) {
                const float lo = v[r], hi = v[r | bit];
                v[r] = lo + hi;
                v[r | bit] = lo - hi;
            }
    // One stage = 8 x (t += s * t of the partner lane), the partner read through DPP inside the multiply-add. The
    // compiler does not fuse the two, and does not see the wait states a DPP read needs after the write of its
    // source (2) or of EXEC (5): the leading s_nop covers both, and inside a block no instruction reads what the one
    // before it wrote through DPP.
#define T3_ROW16_STAGE(CTRL, SIGN)                                                                     \
    asm("s_nop 4\n\t"                                                                                  \
        "v_fmac_f32_dpp %0, %0, %8 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                            \
        "v_fmac_f32_dpp %1, %1, %8 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                            \
        "v_fmac_f32_dpp %2, %2, %8 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                            \
        "v_fmac_f32_dpp %3, %3, %8 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                            \
        "v_fmac_f32_dpp %4, %4, %8 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                            \
        "v_fmac_f32_dpp %5, %5, %8 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                            \
        "v_fmac_f32_dpp %6, %6, %8 " CTRL " row_mask:0xf bank_mask:0xf\n\t"                            \
        "v_fmac_f32_dpp %7, %7, %8 " CTRL " row_mask:0xf bank_mask:0xf"                                 \
        : "+v"(v[0]), "+v"(v[1]), "+v"(v[2]), "+v"(v[3]), "+v"(v[4]), "+v"(v[5]), "+v"(v[6]), "+v"(v[7]) \
        : "v"(SIGN))
    T3_ROW16_STAGE("quad_perm:[1,0,3,2]", g.s1);
    T3_ROW16_STAGE("quad_perm:[2,3,0,1]", g.s2);
    {
        // lane q ^ 4 is q + 4 for the lanes of groups 0 and 2 (row_ror:12 reads lane q - 12 = q + 4 mod 16), q - 4 for
        // groups 1 and 3: two masked moves fill one register with the partners, then the multiply-adds
        float p[8];
        asm("s_nop 4\n\t"
            "v_mov_b32_dpp %0, %8 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
            "v_mov_b32_dpp %1, %9 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
            "v_mov_b32_dpp %2, %10 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
            "v_mov_b32_dpp %3, %11 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
            "v_mov_b32_dpp %4, %12 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
            "v_mov_b32_dpp %5, %13 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
            "v_mov_b32_dpp %6, %14 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
            "v_mov_b32_dpp %7, %15 row_ror:12 row_mask:0xf bank_mask:0x5\n\t"
            "v_mov_b32_dpp %0, %8 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
            "v_mov_b32_dpp %1, %9 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
            "v_mov_b32_dpp %2, %10 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
            "v_mov_b32_dpp %3, %11 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
            "v_mov_b32_dpp %4, %12 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
            "v_mov_b32_dpp %5, %13 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
            "v_mov_b32_dpp %6, %14 row_ror:4 row_mask:0xf bank_mask:0xa\n\t"
            "v_mov_b32_dpp %7, %15 row_ror:4 row_mask:0xf bank_mask:0xa"
            : "=&v"(p[0]), "=&v"(p[1]), "=&v"(p[2]), "=&v"(p[3]), "=&v"(p[4]), "=&v"(p[5]), "=&v"(p[6]), "=&v"(p[7])
            : "v"(v[0]), "v"(v[1]), "v"(v[2]), "v"(v[3]), "v"(v[4]), "v"(v[5]), "v"(v[6]), "v"(v[7]));
#pragma unroll
        for (uint32_t r = 0; r < 8u; ++r) v[r] = __builtin_fmaf(g.s4, p[r], v[r]);
    }
    T3_ROW16_STAGE("row_ror:8", g.s8);
#undef T3_ROW16_STAGE
}

// prepare: the lane's 8 scaled inputs -> its prepared f16 values, elements 2p and 2p + 1 packed in hv[p]; sum: the
// block's sum of the prepared values, valid in the block's lane q = 0 (want_sum false: not computed, 0)
__device__ __forceinline__ void prep_row16(float (&v)[8], const Row16& g, uint32_t (&hv)[4], float& sum, bool want_sum) {
    h128_row16(v, g);
    uint32_t h[8];
#pragma unroll
    for (uint32_t r = 0; r < 8u; ++r) h[r] = half_bits(v[r] * g.scale);
#pragma unroll
    for (uint32_t p = 0; p < 4u; ++p) hv[p] = h[2u * p] | (h[2u * p + 1u] << 16);
    sum = 0.0f;
    if (!want_sum) return;
#pragma unroll
    for (uint32_t r = 0; r < 8u; ++r) sum += half_value(h[r]);
    sum += dpp_take<kDppXor1>(sum);
    sum += dpp_take<kDppXor2>(sum);
    sum += dpp_take<kDppRor4>(sum);
    sum += dpp_take<kDppRor8>(sum);
}

// finish: the lane's 8 sums (through the deferred map when there is one) and svh values -> the finished values
__device__ __forceinline__ void finish_row16(float (&s)[8], const float (&sv)[8], const Row16& g) {
    float v[8];
#pragma unroll
    for (uint32_t r = 0; r < 8u; ++r) v[r] = round_half(s[r]);
    h128_row16(v, g);
#pragma unroll
    for (uint32_t r = 0; r < 8u; ++r) s[r] = round_half(v[r] * g.scale * sv[r]);
}

__device__ __forceinline__ void finish_row16_glm(float (&s)[8], const float (&sv)[8], const Row16& g, bool to_bf16) {
    h128_row16(s, g);
#pragma unroll
    for (uint32_t r = 0; r < 8u; ++r) {
        s[r] = s[r] * g.scale * sv[r];
        if (to_bf16) s[r] = round_bf16(s[r]);
    }
}

// 8 adjacent values from element i (a multiple of 8) of an array whose base is 16-byte aligned
__device__ __forceinline__ void load8_half(const uint16_t* p, size_t i, float (&o)[8]) {
    const uint4v w = *reinterpret_cast<const uint4v*>(p + i);
#pragma unroll
    for (uint32_t k = 0; k < 4u; ++k) {
        o[2u * k] = half_value(w[k] & 0xFFFFu);
        o[2u * k + 1u] = half_value(w[k] >> 16);
    }
}
// 0 + p[0] + p[1] + ... + p[count - 1] in that order, the same value in every lane: up to 64 terms come with one load across
// the wave's lanes (one round trip, not one a term) and are added lane by lane; more go one by one.
__device__ __forceinline__ float wave_ordered_sum(const float* p, uint32_t count, uint32_t lane) {
    float acc = 0.0f;
    if (count <= 64u) {
        const float mine = lane < count ? p[lane] : 0.0f;
        for (uint32_t q = 0; q < count; ++q)
            acc += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mine), static_cast<int>(q)));
    } else {
        for (uint32_t q = 0; q < count; ++q) acc += p[q];
    }
    return acc;
}

// Eight adjacent sums of a GEMM's output plane: f32, or already rounded to f16 where the plane is the chain's z itself
// (one K part and no deferred map: the rounding the finish would start with was done at the GEMM's end).
__device__ __forceinline__ void load8_f32(const float* p, size_t i, float (&o)[8]);
__device__ __forceinline__ void load8_half(const uint16_t* p, size_t i, float (&o)[8]);
__device__ __forceinline__ void load8_plane(const float* p, size_t i, bool half, float (&o)[8]) {
    if (half) load8_half(reinterpret_cast<const uint16_t*>(p), i, o);
    else load8_f32(p, i, o);
}
__device__ __forceinline__ void load8_f32(const float* p, size_t i, float (&o)[8]) {
    const float4v a = *reinterpret_cast<const float4v*>(p + i), b = *reinterpret_cast<const float4v*>(p + i + 4);
#pragma unroll
    for (uint32_t k = 0; k < 4u; ++k) {
        o[k] = a[k];
        o[4u + k] = b[k];
    }
}
template <int DT>
__device__ __forceinline__ void load8_act(const void* p, size_t i, float (&o)[8]) {
    if constexpr (DT == kF32) {
        load8_f32(static_cast<const float*>(p), i, o);
    } else if constexpr (DT == kF16) {
        load8_half(static_cast<const uint16_t*>(p), i, o);
    } else {
        const uint4v w = *reinterpret_cast<const uint4v*>(static_cast<const uint16_t*>(p) + i);
#pragma unroll
        for (uint32_t k = 0; k < 4u; ++k) {
            o[2u * k] = bf16_value(static_cast<uint16_t>(w[k] & 0xFFFFu));
            o[2u * k + 1u] = bf16_value(static_cast<uint16_t>(w[k] >> 16));
        }
    }
}
template <int DT>
__device__ __forceinline__ void store8_act(void* p, size_t i, const float (&v)[8]) {
    if constexpr (DT == kF32) {
        float* f = static_cast<float*>(p) + i;
        *reinterpret_cast<float4v*>(f) = float4v{v[0], v[1], v[2], v[3]};
        *reinterpret_cast<float4v*>(f + 4) = float4v{v[4], v[5], v[6], v[7]};
    } else {
        uint4v w;
#pragma unroll
        for (uint32_t k = 0; k < 4u; ++k) {
            const uint32_t lo = DT == kF16 ? half_bits(v[2u * k]) : bf16_bits(v[2u * k]);
            const uint32_t hi = DT == kF16 ? half_bits(v[2u * k + 1u]) : bf16_bits(v[2u * k + 1u]);
            w[k] = lo | (hi << 16);
        }
        *reinterpret_cast<uint4v*>(static_cast<uint16_t*>(p) + i) = w;
    }
}
__device__ __forceinline__ void load8_act_rt(int dt, const void* p, size_t i, float (&o)[8]) {
    if (dt == kF32) load8_act<kF32>(p, i, o);
    else if (dt == kF16) load8_act<kF16>(p, i, o);
    else load8_act<kBf16>(p, i, o);
}
__device__ __forceinline__ void store8_act_rt(int dt, void* p, size_t i, const float (&v)[8]) {
    if (dt == kF32) store8_act<kF32>(p, i, v);
    else if (dt == kF16) store8_act<kF16>(p, i, v);
    else store8_act<kBf16>(p, i, v);
}

// the lane's four packed pairs of prepared values into f16 [..] in pair-quad order: block b of the row at row_at,
// elements 8 q + 2p, + 1 (pair_quad_slot of t3_common.hpp, for a lane's 8 elements at once)
__device__ __forceinline__ void store_pair_quad(uint16_t* base, size_t row_at, uint32_t b, uint32_t q, const uint32_t (&hv)[4]) {
    uint32_t* w = reinterpret_cast<uint32_t*>(base + row_at + b * 128u + 32u * (q >> 2) + 4u * ((q >> 1) & 1u) + 2u * (q & 1u));
#pragma unroll
    for (uint32_t p = 0; p < 4u; ++p) w[4u * p] = hv[p];
}

}  // namespace t3
