// The wave64 trellis reader and the two codebooks.
//
// A packed tile holds 256 codewords in "code position" order; weight t's codeword is the 16-bit window of the tile's
// circular MSB-first bitstream that ends at bit ((t + 1) n) >> 4, n the tile's halfwords (turboexl3
// src/core/format.zig:176-222). Position p = 8 L + i maps to tile row 2 (L % 4) + {0, 1, 8, 9}[i % 4] and column
// L / 4 + 8 (i / 4) (format.zig:237-256).
//
// One wave64 reads one tile, four consecutive positions a lane ("a quad"): lane l, with c = l % 16 and g = l / 16,
// takes positions P..P+3, P = 8 (4 (c % 8) + g) + 4 (c / 8): the weights of output column c at input rows
// 2g + {0, 1, 8, 9}. That is the A fragment of v_mfma_f32_16x16x32_f16 when every weight fills a pair of K slots
// (M = column c = l % 16, K slots 8g..8g+7), so decoded registers feed the matrix core with no shuffle.
//
// A quad's four windows span at most 3n/16 + 17 bits. Up to n = 84 they fit one 32-bit register R (the 32 stream bits
// ending at the last window's end): two word loads, one v_alignbit, one v_bfe a weight (kNarrow). Wider rates read the
// first two windows from a second register ending at window 1's end: cut from the same two words where every quad's
// span lies inside them (kWidePair: n = 86..90, 96, 128), from two more words otherwise (kWide).
#pragma once

#include <type_traits>

#include "t3_common.hpp"

namespace t3 {

// format.zig Codebook's numbering, extended with the two GEMV-only forms
enum Codebook : int {
    kMul1 = 0,      // exact f16 weight, fma(f16(1024 + t), A, B)
    kMcg = 1,       // exact f16 weight, f16(lo + hi)
    kMul1Defer = 2, // h = 1024 + t as the weight; the affine map applied once an output (A acc + B sum x)
    kMcgPair = 3,   // the hashed pair (lo, hi) as two K slots: x lo + x hi, the weight never rounded to f16
    kMcgTab = 4,    // kMcg's weights, some of a lane's looked up in an LDS table of all 65,536 (the measured two-pipe
                    // form: t3_dense.hip, dense_gemv_tab)
};

constexpr uint32_t kMcgMult = 0xCBAC1FEDu;
constexpr uint32_t kMul1Mult = 0x83DCD12Du;

// cw times a 32-bit constant, modulo 2^32. v_mul_lo_u32 issues at the full VALU rate on gfx950 (measured: the same
// lane-ops/s as v_mul_u32_u24), so the one-instruction form beats any split over the 24-bit multiplier.
template <uint32_t M>
__device__ __forceinline__ uint32_t hash_mul(uint32_t cw) {
    return cw * M;
}

// MUL1's h = 0x6400 + byte sum of the hashed codeword: the f16 bit pattern of 1024 + t, t in [0, 1020]
__device__ __forceinline__ uint32_t mul1_h(uint32_t cw) {
    return __builtin_amdgcn_sad_u8(hash_mul<kMul1Mult>(cw), 0u, 0x6400u);
}
__device__ __forceinline__ uint32_t mul1_t(uint32_t cw) { return mul1_h(cw) - 0x6400u; }

// MCG's hashed pair: two f16 with fixed exponent range, sign and mantissa from the hash
__device__ __forceinline__ uint32_t mcg_pair(uint32_t cw) {
    return 0x3B603B60u ^ (hash_mul<kMcgMult>(cw) & 0x8FFF8FFFu);
}

// Exact decoders (format.zig:149-167). MCG: both halves have exponents in [2^-3, 2^0], so their f32 sum is exact and
// one f16 add rounds as f16(f32(lo) + f32(hi)) does. MUL1: (1024 + t) A + B is a multiple of 2^-18 below 4, exact in
// f32, so one fused f16 multiply-add rounds as f16(fmaf(...)) does.
__device__ __forceinline__ uint16_t decode_mcg(uint32_t cw) {
    const uint32_t p = mcg_pair(cw);
    const _Float16 lo = __builtin_bit_cast(_Float16, static_cast<uint16_t>(p & 0xFFFFu));
    const _Float16 hi = __builtin_bit_cast(_Float16, static_cast<uint16_t>(p >> 16));
    return __builtin_bit_cast(uint16_t, static_cast<_Float16>(lo + hi));
}
__device__ __forceinline__ uint16_t decode_mul1(uint32_t cw) {
    const _Float16 h = __builtin_bit_cast(_Float16, static_cast<uint16_t>(mul1_h(cw)));
    const _Float16 a = __builtin_bit_cast(_Float16, static_cast<uint16_t>(0x1EEEu));
    const _Float16 b = __builtin_bit_cast(_Float16, static_cast<uint16_t>(0xC931u));
    return __builtin_bit_cast(uint16_t, __builtin_fmaf16(h, a, b));
}
template <int CB>
__device__ __forceinline__ uint16_t decode_exact(uint32_t cw) {
    if constexpr (CB == kMcg || CB == kMcgPair || CB == kMcgTab) return decode_mcg(cw);
    else return decode_mul1(cw);
}

// A weight as the GEMV's matrix core takes it: 32 bits = two f16 K slots (the second zero unless kMcgPair).
template <int CB>
__device__ __forceinline__ uint32_t weight_pair(uint32_t cw) {
    if constexpr (CB == kMcgPair) return mcg_pair(cw);
    else if constexpr (CB == kMul1Defer) return mul1_h(cw);
    else return static_cast<uint32_t>(decode_exact<CB>(cw));
}

// The weight the matrix core takes as one f16 (the GEMMs, and the GEMV's two-tile-row steps): exact, or MUL1's h = 1024 + t when its map is deferred.
template <int CB>
__device__ __forceinline__ uint32_t weight_half(uint32_t cw) {
    if constexpr (CB == kMul1Defer) return mul1_h(cw);
    else return static_cast<uint32_t>(decode_exact<CB>(cw));
}

// Two weights as the two halves of one register. MCG: each weight is one f16 add of its hashed pair's halves, and the
// sub-dword forms of v_add_f16 write the low half, then the high half of the same register (the plain form costs a
// third instruction to merge them).
template <int CB>
__device__ __forceinline__ uint32_t weight_halves(uint32_t cw_lo, uint32_t cw_hi) {
    if constexpr (CB == kMcg) {
        const uint32_t pa = mcg_pair(cw_lo), pb = mcg_pair(cw_hi);
        uint32_t d;
        asm("v_add_f16_sdwa %0, %1, %1 dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:WORD_0 src1_sel:WORD_1"
            : "=v"(d)
            : "v"(pa));
        // the two wait states a sub-dword write needs before a matrix instruction reads the register: the compiler
        // adds them for its own SDWA instructions, not for this one. (The second add keeps the first one's half of d, so
        // it reads d: a sub-dword write wants one wait state before such a read as well. The two adds are separate
        // statements so that the compiler can put the second weight's hash between them, which it does in every
        // kernel compiled from this tree: no pair is adjacent in their ISA. A change that made them adjacent would show
        // as wrong low halves in every parity test that decodes MCG through a GEMV or a GEMM.)
        asm("v_add_f16_sdwa %0, %1, %1 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_0 src1_sel:WORD_1\n\t"
            "s_nop 1"
            : "+v"(d)
            : "v"(pb));
        return d;
    } else {
        return weight_half<CB>(cw_lo) | (weight_half<CB>(cw_hi) << 16);
    }
}

// The LDS table form: the f16 weight of every 16-bit codeword at byte 2 cw of the workgroup's dynamic LDS (the kernel
// fills it and keeps no static LDS, so the table starts at LDS address 0). Two weights as one register's halves.
extern __shared__ __attribute__((aligned(16))) unsigned char t3_table_lds[];
__device__ __forceinline__ uint32_t table_halves(uint32_t cw_lo, uint32_t cw_hi) {
    const uint16_t* tab = reinterpret_cast<const uint16_t*>(t3_table_lds);
    return static_cast<uint32_t>(tab[cw_lo]) | (static_cast<uint32_t>(tab[cw_hi]) << 16);
}

// ---- the quad plan --------------------------------------------------------------------------------------------

__device__ __forceinline__ uint32_t quad_first_position(uint32_t lane) {
    const uint32_t c = lane & 15u, g = lane >> 4;
    return 8u * (4u * (c & 7u) + g) + 4u * (c >> 3);
}

// How a lane reads its quad at rate n.
enum Reader : int { kNarrow = 0, kWide = 1, kWidePair = 2 };

// Whether some quad's four windows overflow one 32-bit register at rate n (host and device agree on this rule).
__host__ __device__ inline bool quad_needs_wide(uint32_t n) {
    for (uint32_t q = 0; q < 64u; ++q) {
        const uint32_t e0 = ((4u * q + 1u) * n) >> 4, e3 = ((4u * q + 4u) * n) >> 4;
        if (e3 - e0 > 16u) return true;
    }
    return false;
}
// Whether every quad's four windows lie inside the two words that hold the 32 stream bits ending at window 3's end.
__host__ __device__ inline bool quad_in_two_words(uint32_t n) {
    for (uint32_t q = 0; q < 64u; ++q) {
        const uint32_t e0 = ((4u * q + 1u) * n) >> 4, e3 = ((4u * q + 4u) * n) >> 4;
        const uint32_t w = (e3 + 16u * n - 1u) >> 5;  // one period added, as the plan does
        if (e0 + 16u * n - 16u < 32u * (w - 1u)) return false;
    }
    return true;
}
__host__ __device__ inline int quad_reader(uint32_t n) {
    return !quad_needs_wide(n) ? kNarrow : quad_in_two_words(n) ? kWidePair : kWide;
}

// Host side: call f with the rate's reader as a compile-time constant.
template <typename F>
inline auto with_reader(uint32_t n, F&& f) {
    switch (quad_reader(n)) {
        case kWide: return f(std::integral_constant<int, kWide>{});
        case kWidePair: return f(std::integral_constant<int, kWidePair>{});
        default: return f(std::integral_constant<int, kNarrow>{});
    }
}

template <int WIDE>
struct QuadPlan {
    uint32_t ib_prev, ib_last, shb;  // register B: the 32 stream bits ending at window 3's end
    uint32_t ia_prev, ia_last, sha;  // register A (wide readers): ... ending at window 1's end
    uint32_t a_low;                  // kWidePair: register A's low word is B's previous word (else B's last)
    uint32_t o[4];                   // window m's right shift inside its register
};

template <int WIDE>
__device__ __forceinline__ QuadPlan<WIDE> quad_plan(uint32_t n, uint32_t lane) {
    const uint32_t p = quad_first_position(lane);
    const uint32_t nw = n >> 1, total = 16u * n;
    uint32_t e[4];
#pragma unroll
    for (uint32_t m = 0; m < 4u; ++m) e[m] = ((p + m + 1u) * n) >> 4;
    QuadPlan<WIDE> q;
    {
        // one period added keeps the word index positive: w is in [nw, 2 nw), so the modulo is one subtraction
        const uint32_t end = e[3] + total;
        const uint32_t w = (end - 1u) >> 5;
        q.shb = 32u * (w + 1u) - end;
        q.ib_last = w - nw;
        q.ib_prev = w - 1u >= nw ? w - 1u - nw : w - 1u;
    }
    q.a_low = 0u;
    if constexpr (WIDE == kWidePair) {
        // the 64 bits {previous, last} shifted right until window 1's end is bit 0: by less than 32, one v_alignbit of
        // the pair; by 32 or more, the previous word alone (its own bits fill the top, above the two windows)
        const uint32_t sa = q.shb + (e[3] - e[1]);
        q.a_low = sa >= 32u ? 1u : 0u;
        q.sha = sa & 31u;
        q.ia_last = q.ia_prev = 0u;
        q.o[0] = e[1] - e[0];
        q.o[1] = 0u;
        q.o[2] = e[3] - e[2];
        q.o[3] = 0u;
    } else if constexpr (WIDE == kWide) {
        const uint32_t end = e[1] + total;
        const uint32_t w = (end - 1u) >> 5;
        q.sha = 32u * (w + 1u) - end;
        q.ia_last = w - nw;
        q.ia_prev = w - 1u >= nw ? w - 1u - nw : w - 1u;
        q.o[0] = e[1] - e[0];
        q.o[1] = 0u;
        q.o[2] = e[3] - e[2];
        q.o[3] = 0u;
    } else {
        q.sha = q.ia_last = q.ia_prev = 0u;
#pragma unroll
        for (uint32_t m = 0; m < 4u; ++m) q.o[m] = e[3] - e[m];
    }
    return q;
}

// The words a lane holds of one tile, loaded ahead of their use.
template <int WIDE>
struct QuadWords {
    uint32_t b_prev, b_last, a_prev, a_last;  // the a words: kWide only
};

template <int WIDE>
__device__ __forceinline__ QuadWords<WIDE> quad_load(const uint32_t* tile, const QuadPlan<WIDE>& q) {
    QuadWords<WIDE> w;
    w.b_prev = tile[q.ib_prev];
    w.b_last = tile[q.ib_last];
    if constexpr (WIDE == kWide) {
        w.a_prev = tile[q.ia_prev];
        w.a_last = tile[q.ia_last];
    } else {
        w.a_prev = w.a_last = 0u;
    }
    return w;
}

// The quad's four codewords, masked to the pack's window width `wbits` (8..16).
template <int WIDE>
__device__ __forceinline__ void quad_codewords(const QuadWords<WIDE>& w, const QuadPlan<WIDE>& q, uint32_t wbits,
                                               uint32_t (&cw)[4]) {
    const uint32_t rb = __builtin_amdgcn_alignbit(w.b_prev, w.b_last, q.shb);
    uint32_t ra = rb;
    if constexpr (WIDE == kWide) ra = __builtin_amdgcn_alignbit(w.a_prev, w.a_last, q.sha);
    if constexpr (WIDE == kWidePair) ra = __builtin_amdgcn_alignbit(w.b_prev, q.a_low ? w.b_prev : w.b_last, q.sha);
    cw[0] = __builtin_amdgcn_ubfe(ra, q.o[0], wbits);
    cw[1] = __builtin_amdgcn_ubfe(ra, q.o[1], wbits);
    cw[2] = __builtin_amdgcn_ubfe(rb, q.o[2], wbits);
    cw[3] = __builtin_amdgcn_ubfe(rb, q.o[3], wbits);
}

// Tile row of a quad's weight m, and its column: the inverse of the permutation for one lane.
__device__ __forceinline__ uint32_t quad_row(uint32_t lane, uint32_t m) {
    return 2u * (lane >> 4) + (m & 1u) + 8u * (m >> 1);
}
__device__ __forceinline__ uint32_t quad_col(uint32_t lane) { return lane & 15u; }

}  // namespace t3
