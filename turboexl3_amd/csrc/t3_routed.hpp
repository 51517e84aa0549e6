// Device helpers shared by the routed kernels at decode rows and at prefill: a row-slot's expert, its score, and the
// sum of a block's K-slice planes.
#pragma once

#include "t3_common.hpp"
#include "t3_kernels.hpp"
#include "t3_stages.hpp"

namespace t3 {

struct SlotRef {
    uint32_t row, e;
    bool live, shared;
};

// Row-slot rk of KT = topk + shared slots a row. A routed id outside [0, experts) is skipped, as the reference skips it
// (src/kernels/hip/decode/decode.hip:26-28).
__device__ __forceinline__ SlotRef resolve_slot(const MoeLaunch& a, uint32_t rk) {
    SlotRef s;
    const uint32_t kt = a.topk + a.shared_slots;
    s.row = rk / kt;
    const uint32_t k = rk - s.row * kt;
    s.shared = k >= a.topk;
    if (s.shared) {
        s.e = k - a.topk;
        s.live = true;
    } else {
        const int32_t es = a.slots[s.row * a.topk + k];
        s.live = es >= 0 && static_cast<uint32_t>(es) < a.bank.experts;
        s.e = static_cast<uint32_t>(es);
    }
    return s;
}

__device__ __forceinline__ float score_of(const MoeLaunch& a, uint32_t row, uint32_t k) {
    const size_t i = static_cast<size_t>(row) * a.topk + k;
    if (a.score_dt == kF32) return static_cast<const float*>(a.scores)[i];
    if (a.score_dt == kF16) return half_value(static_cast<const uint16_t*>(a.scores)[i]);
    return bf16_value(static_cast<const uint16_t*>(a.scores)[i]);
}

// The gated shared expert's arithmetic lives in the activation dtype (f16 or bf16), one rounding an operation, as the
// host's chain of MLX operations it stands for (src/models/qwen38/kernels/shared/shared_fin_head_4.metal:1-9,
// dfin7s.metal:44-50).
__device__ __forceinline__ float round_act(int dt, float v) {
    return dt == kF16 ? round_half(v) : (dt == kBf16 ? bf16_value(bf16_bits(v)) : v);
}
// sigtab's entry for the 16-bit pattern of v (already a value of the dtype)
__device__ __forceinline__ float sigmoid_of(const MoeLaunch& a, float v) {
    const uint32_t bits = a.dtype == kF16 ? half_bits(v) : bf16_bits(v);
    const uint16_t t = static_cast<const uint16_t*>(a.sigtab)[bits];
    return a.dtype == kF16 ? half_value(t) : bf16_value(t);
}
// h = ((g * sigmoid(g)) * u), every step in the dtype
__device__ __forceinline__ float swiglu_table(const MoeLaunch& a, float g, float u) {
    const float gt = round_act(a.dtype, g), ut = round_act(a.dtype, u);
    const float act = round_act(a.dtype, gt * sigmoid_of(a, gt));
    return round_act(a.dtype, act * ut);
}
// the shared slot's term of a row's output: sigmoid(logit[row]) * dtype(v), in the dtype
__device__ __forceinline__ float gated_term(const MoeLaunch& a, uint32_t row, float v) {
    const float logit = load_act_rt(a.dtype, a.slogit, row);
    return round_act(a.dtype, sigmoid_of(a, logit) * round_act(a.dtype, v));
}

// One block's sums over the K slices (slice order; the first plane starts the sum) and the deferred MUL1 map.
// COH: the planes and block sums were stored by other workgroups of this launch.
// Loads go out eight at a time and are added in slice (or block) order: the sums do not depend on the batching, and a
// block's finish waits for one round trip, not for one a plane.
template <bool COH>
__device__ __forceinline__ float ordered_sum(const float* p, size_t stride, uint32_t count, bool first_starts) {
    auto get = [](const float* q) { return COH ? load_coherent(q) : *q; };
    float acc = 0.0f;
    for (uint32_t k0 = 0; k0 < count; k0 += 8u) {
        float part[8];
#pragma unroll
        for (uint32_t k = 0; k < 8u; ++k) part[k] = k0 + k < count ? get(p + (k0 + k) * stride) : 0.0f;
#pragma unroll
        for (uint32_t k = 0; k < 8u; ++k)
            if (k0 + k < count) acc = first_starts && k0 + k == 0u ? part[k] : acc + part[k];  // 0 + z would turn -0 into +0
    }
    return acc;
}

// N such sums at once: every load of all of them goes out before the first add (up to 8 planes; more fall back to one
// sum after the other). The same order of additions a sum as ordered_sum's.
template <bool COH, int N>
__device__ __forceinline__ void ordered_sums(const float* const (&p)[N], size_t stride, uint32_t count, float (&out)[N]) {
    auto get = [](const float* q) { return COH ? load_coherent(q) : *q; };
    if (count <= 8u) {
        float part[N][8];
#pragma unroll
        for (int i = 0; i < N; ++i)
#pragma unroll
            for (uint32_t k = 0; k < 8u; ++k) part[i][k] = k < count ? get(p[i] + k * stride) : 0.0f;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            float acc = part[i][0];
#pragma unroll
            for (uint32_t k = 1; k < 8u; ++k)
                if (k < count) acc += part[i][k];
            out[i] = acc;
        }
    } else {
#pragma unroll
        for (int i = 0; i < N; ++i) out[i] = ordered_sum<COH>(p[i], stride, count, true);
    }
}

// Whether the launch's codebook form defers MUL1's map: known when the kernel is compiled (DEFER 0 or 1: the GEMV
// kernels, whose codebook form is a template argument, carry no code of the other case) or read from the launch (-1).
template <int DEFER>
__device__ __forceinline__ bool defers(const MoeLaunch& a) {
    if constexpr (DEFER < 0) return a.defer != 0;
    else return DEFER != 0;
}

// 0 + p[0] + p[1] + ... in that order, the values fetched by one load across the wave's lanes (up to 64 of them)
// In two steps, so that a caller can send the load out beside its other loads and add up once they are all back:
// lane_sum_fetch is the load (a lane's own value), lane_sum_fold the additions.
template <bool COH>
__device__ __forceinline__ float lane_sum_fetch(const float* p, uint32_t count, uint32_t lane) {
    return lane < count ? (COH ? load_coherent(p + lane) : p[lane]) : 0.0f;
}
template <bool COH>
__device__ __forceinline__ float lane_sum_fold(float mine, const float* p, uint32_t count) {
    if (count > 64u) return ordered_sum<COH>(p, 1u, count, false);
    float acc = 0.0f;
    for (uint32_t q = 0; q < count; ++q)
        acc += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, mine), static_cast<int>(q)));
    return acc;
}
template <bool COH>
__device__ __forceinline__ float lane_ordered_sum(const float* p, uint32_t count, uint32_t lane) {
    return lane_sum_fold<COH>(lane_sum_fetch<COH>(p, count, lane), p, count);
}

template <bool COH>
__device__ __forceinline__ void plane_sums(const float* z, size_t planes_stride, uint32_t ks, const float* bsum,
                                           uint32_t nb, int defer, uint32_t lane, float (&s)[2]) {
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) s[j] = ordered_sum<COH>(z + lane + 64u * j, planes_stride, ks, true);
    if (defer) {
        const float xsum = ordered_sum<COH>(bsum, 1u, nb, false);
#pragma unroll
        for (uint32_t j = 0; j < 2u; ++j) s[j] = __builtin_fmaf(s[j], mul1_a(), mul1_b() * xsum);
    }
}

// ---- the routed chain's per-block stages ----------------------------------------------------------------------
// One wave a 128-block. rk: the row-slot; q: where its scratch lives (decode rows: q = rk; prefill: its position in
// the expert-sorted order). PF = prefill: the prepared activations are plain f16 (the GEMM's B fragments), one plane a
// projection; else ks planes, and the activations as the GEMV's codebook form reads them (a.pair_order: plain f16 in
// pair-quad order as well, two tile rows a step; else u32 with the f16 in both halves, the pairs of K slots).

template <bool PF>
__device__ __forceinline__ void store_prepared(const MoeLaunch& a, uint32_t* base, size_t row_at, uint32_t i, uint32_t hbits) {
    if (PF || a.pair_order) reinterpret_cast<uint16_t*>(base)[row_at + pair_quad_slot(i)] = static_cast<uint16_t>(hbits);
    else base[row_at + (i & ~15u) + quad_slot(i & 15u)] = hbits | (hbits << 16);
}

// the gate's and the up's prepare of block b of row-slot rk: xg, xu [.][hidden], sg, su [.][hidden / 128]
template <bool PF, int PROF = 0>
__device__ __forceinline__ void routed_prep_block(const MoeLaunch& a, uint32_t rk, uint32_t q, uint32_t b,
                                                  uint32_t lane) {
    const SlotRef s = resolve_slot(a, rk);
    if (!s.live) return;
    const RoutedBank& bank = s.shared ? a.shared : a.bank;
    const uint32_t nb = a.hidden / 128u;
#pragma unroll
    for (uint32_t proj = 0; proj < 2u; ++proj) {
        const uint16_t* suh = (proj ? bank.up_suh : bank.gate_suh) + static_cast<size_t>(s.e) * a.hidden;
        uint32_t hv[2];
        float sum;
        prep_values(a.dtype, a.x, suh, a.hidden, s.row, b, lane, hv, sum, PROF == 0);
#pragma unroll
        for (uint32_t j = 0; j < 2u; ++j)
            store_prepared<PF>(a, proj ? a.xu : a.xg, static_cast<size_t>(q) * a.hidden, b * 128u + lane + 64u * j, hv[j]);
        if (lane == 0u) (proj ? a.su : a.sg)[static_cast<size_t>(q) * nb + b] = sum;
    }
}

// gate and up finishes, the (clamped) SwiGLU in f32 on their f16 values, and the down's prepare: hd [.][inter],
// hs f32 [.][inter / 128]
// the values of it: hh[j], the prepared f16 of element lane + 64 j of the block, and the block's sum of them
template <bool PF, bool COH = false, int PROF = 0, int DEFER = -1>
__device__ __forceinline__ void routed_mid_values(const MoeLaunch& a, const SlotRef& s, uint32_t q, uint32_t b,
                                                  uint32_t lane, uint32_t (&hh)[2], float& sum) {
    const RoutedBank& bank = s.shared ? a.shared : a.bank;
    const uint32_t rkt = a.rows * (a.topk + a.shared_slots), nb = a.hidden / 128u;
    const uint32_t ks = PF ? 1u : a.ks_gu;
    const size_t plane = static_cast<size_t>(rkt) * a.inter, at = static_cast<size_t>(q) * a.inter + b * 128u;
    // every load of the block goes out together: one round trip, not one a plane and a projection
    const size_t eo = static_cast<size_t>(s.e) * a.inter + b * 128u;
    float svg[2], svu[2], sdn[2];
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
        svg[j] = half_value(bank.gate_svh[eo + lane + 64u * j]);
        svu[j] = half_value(bank.up_svh[eo + lane + 64u * j]);
        sdn[j] = half_value(bank.down_suh[eo + lane + 64u * j]);
    }
    const float* const planes[4] = {a.zg + at + lane, a.zg + at + lane + 64u, a.zu + at + lane, a.zu + at + lane + 64u};
    float sums[4];
    const float* sgp = a.sg + static_cast<size_t>(q) * nb;
    const float* sup = a.su + static_cast<size_t>(q) * nb;
    const bool defer = defers<DEFER>(a);
    const float mg = defer ? lane_sum_fetch<COH>(sgp, nb, lane) : 0.0f;  // out with the planes' loads
    const float mu = defer ? lane_sum_fetch<COH>(sup, nb, lane) : 0.0f;
    ordered_sums<COH, 4>(planes, plane, ks, sums);
    float g[2] = {sums[0], sums[1]}, u[2] = {sums[2], sums[3]};
    if (defer) {
        const float xg = lane_sum_fold<COH>(mg, sgp, nb);
        const float xu = lane_sum_fold<COH>(mu, sup, nb);
#pragma unroll
        for (uint32_t j = 0; j < 2u; ++j) {
            g[j] = __builtin_fmaf(g[j], mul1_a(), mul1_b() * xg);
            u[j] = __builtin_fmaf(u[j], mul1_a(), mul1_b() * xu);
        }
    }
    float d[2];
    if constexpr (PROF == 0) {
        finish_core(g, svg, lane);
        finish_core(u, svu, lane);
#pragma unroll
        for (uint32_t j = 0; j < 2u; ++j) {
            const float h = s.shared && a.sigtab ? swiglu_table(a, g[j], u[j]) : swiglu_clamped(g[j], u[j], a.limit, a.clamp_at);
            d[j] = round_half(h) * sdn[j];
        }
    } else {
        finish_core_glm(g, svg, lane, true);
        finish_core_glm(u, svu, lane, true);
#pragma unroll
        for (uint32_t j = 0; j < 2u; ++j) d[j] = swiglu_glm(g[j], u[j], a.limit) * sdn[j];
    }
    h128_wave(d, lane);
    sum = 0.0f;
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
        hh[j] = half_bits(d[j] * kHadScale);
        sum += half_value(hh[j]);
    }
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) sum += __shfl_xor(sum, m, 64);
}

template <bool PF, bool COH = false, int PROF = 0, int DEFER = -1>
__device__ __forceinline__ void routed_mid_block(const MoeLaunch& a, const SlotRef& s, uint32_t q, uint32_t b,
                                                 uint32_t lane) {
    if (!s.live) return;
    uint32_t hh[2];
    float sum;
    routed_mid_values<PF, COH, PROF, DEFER>(a, s, q, b, lane, hh, sum);
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j)
        store_prepared<PF>(a, a.hd, static_cast<size_t>(q) * a.inter, b * 128u + lane + 64u * j, hh[j]);
    if (defers<DEFER>(a) && lane == 0u) a.hs[static_cast<size_t>(q) * (a.inter / 128u) + b] = sum;  // the map's alone
}

// One slot's finished down outputs of block b (f16-valued), false for a skipped slot. COH: only the planes cross
// workgroups inside the launch; the block sums hs came from the launch before.
template <bool COH, bool HS_COH = false, int PROF = 0>
__device__ __forceinline__ bool routed_down_finish(const MoeLaunch& a, const SlotRef& s, uint32_t q, uint32_t b,
                                                   uint32_t lane, float (&v)[2], uint32_t ks) {
    if (!s.live) return false;  // uniform over the wave
    const uint32_t rkt = a.rows * (a.topk + a.shared_slots), nbi = a.inter / 128u;
    const RoutedBank& bank = s.shared ? a.shared : a.bank;
    const float* z = a.zd + static_cast<size_t>(q) * a.hidden + b * 128u;
    const size_t plane = static_cast<size_t>(rkt) * a.hidden;
    // the block's scales go out with the planes, not after them
    const uint16_t* svh = bank.down_svh + static_cast<size_t>(s.e) * a.hidden + b * 128u;
    const float sv[2] = {half_value(svh[lane]), half_value(svh[lane + 64u])};
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) v[j] = ordered_sum<COH>(z + lane + 64u * j, plane, ks, true);
    if (a.defer) {
        const float xsum = ordered_sum<HS_COH>(a.hs + static_cast<size_t>(q) * nbi, 1u, nbi, false);
#pragma unroll
        for (uint32_t j = 0; j < 2u; ++j) v[j] = __builtin_fmaf(v[j], mul1_a(), mul1_b() * xsum);
    }
    if constexpr (PROF == 0) finish_core(v, sv, lane);
    else finish_core_glm(v, sv, lane, false);
    return true;
}

// R slots' finished down outputs of block b at once (a skipped slot's entry is left alone): all their planes, scales
// and block sums are fetched together. q[r]: where slot r's scratch lives.
template <bool COH, bool HS_COH, int R, int PROF = 0, int DEFER = -1>
__device__ __forceinline__ void routed_down_finish_many(const MoeLaunch& a, const SlotRef (&s)[R], const uint32_t (&q)[R],
                                                        uint32_t b, uint32_t lane, float (&v)[R][2], uint32_t ks) {
    const uint32_t rkt = a.rows * (a.topk + a.shared_slots), nbi = a.inter / 128u;
    const size_t plane = static_cast<size_t>(rkt) * a.hidden;
    const float* planes[2 * R];
    float sv[R][2], sums[2 * R], xsum[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        // a skipped slot reads its own (unwritten) scratch and expert 0's scales: valid memory, values unused
        const RoutedBank& bank = s[r].live && s[r].shared ? a.shared : a.bank;
        const uint16_t* svh = bank.down_svh + static_cast<size_t>(s[r].live ? s[r].e : 0u) * a.hidden + b * 128u;
#pragma unroll
        for (uint32_t j = 0; j < 2u; ++j) {
            sv[r][j] = half_value(svh[lane + 64u * j]);
            planes[2 * r + j] = a.zd + static_cast<size_t>(q[r]) * a.hidden + b * 128u + lane + 64u * j;
        }
    }
    // the block sums' loads go out with the planes' (HS_COH: the sums were made inside this launch, a copy a 128-column
    // block of the output)
    const bool defer = defers<DEFER>(a);
    const float* hs[R];
    float mine[R];
#pragma unroll
    for (int r = 0; r < R; ++r) {
        hs[r] = a.hs + (HS_COH ? (static_cast<size_t>(b) * rkt + q[r]) * hs_copy_stride(a.inter) : static_cast<size_t>(q[r]) * nbi);
        mine[r] = defer ? lane_sum_fetch<HS_COH>(hs[r], nbi, lane) : 0.0f;
    }
    ordered_sums<COH, 2 * R>(planes, plane, ks, sums);
    if (defer)
#pragma unroll
        for (int r = 0; r < R; ++r) xsum[r] = lane_sum_fold<HS_COH>(mine[r], hs[r], nbi);
#pragma unroll
    for (int r = 0; r < R; ++r) {
        if (!s[r].live) continue;  // uniform over the wave
        v[r][0] = sums[2 * r];
        v[r][1] = sums[2 * r + 1];
        if (defer)
#pragma unroll
            for (uint32_t j = 0; j < 2u; ++j) v[r][j] = __builtin_fmaf(v[r][j], mul1_a(), mul1_b() * xsum[r]);
        if constexpr (PROF == 0) finish_core(v[r], sv[r], lane);
        else finish_core_glm(v[r], sv[r], lane, false);
    }
}

// a row's block b from its f32 sums: y's dtype; or two roundings: the routed output rounds to x's dtype, then the add
// of `moeWithShared`'s tensor (src/root.zig:976-984) or of the gated shared expert's term (`gated`, where the call has
// a sigmoid table) rounds again
__device__ __forceinline__ void routed_store_row(const MoeLaunch& a, uint32_t row, uint32_t b, uint32_t lane,
                                                 const float (&acc)[2], const float (&gated)[2]) {
    const bool has_gate = a.sigtab != nullptr;
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
        const size_t o = static_cast<size_t>(row) * a.hidden + b * 128u + lane + 64u * j;
        if (a.shared_add || has_gate) {
            const float r = round_act(a.dtype, acc[j]);
            store_act_rt(a.dtype, a.y, o, r + (has_gate ? gated[j] : load_act_rt(a.dtype, a.shared_add, o)));
        } else {
            store_act_rt(a.dtype, a.y, o, acc[j]);
        }
    }
}

// GLM's profile ends here: each routed slot's down finish as f32 [row-slot][hidden], no score, a skipped slot's output
// left as it is (the host combines the slots and its shared expert; src/kernels/hip/decode/decode.hip:11-13)
template <bool PF>
__device__ __forceinline__ void routed_slots_block(const MoeLaunch& a, uint32_t row, uint32_t b, uint32_t lane) {
    for (uint32_t k = 0; k < a.topk; ++k) {
        const uint32_t rk = row * a.topk + k;
        const SlotRef s = resolve_slot(a, rk);
        if (!s.live) continue;  // uniform over the wave
        float v[2];
        routed_down_finish<false, false, 1>(a, s, PF ? a.inv[rk] : rk, b, lane, v, PF ? 1u : a.ks_dn);
#pragma unroll
        for (uint32_t j = 0; j < 2u; ++j)
            static_cast<float*>(a.y)[static_cast<size_t>(rk) * a.hidden + b * 128u + lane + 64u * j] = v[j];
    }
}

// every slot's down finish of block b of one row, then the score-weighted sum in slot order
template <bool PF>
__device__ __forceinline__ void routed_combine_block(const MoeLaunch& a, uint32_t row, uint32_t b, uint32_t lane) {
    const uint32_t kt = a.topk + a.shared_slots;
    float acc[2] = {0.0f, 0.0f}, gated[2] = {0.0f, 0.0f};
    for (uint32_t k = 0; k < kt; ++k) {
        const uint32_t rk = row * kt + k;
        const SlotRef s = resolve_slot(a, rk);
        if (!s.live) continue;  // uniform over the wave
        float v[2];
        routed_down_finish<false>(a, s, PF ? a.inv[rk] : rk, b, lane, v, PF ? 1u : a.ks_dn);
        if (s.shared && a.sigtab) {
            gated[0] = gated_term(a, row, v[0]);
            gated[1] = gated_term(a, row, v[1]);
            continue;
        }
        const float w = s.shared ? 1.0f : score_of(a, row, k);
#pragma unroll
        for (uint32_t j = 0; j < 2u; ++j) acc[j] = __builtin_fmaf(w, v[j], acc[j]);
    }
    routed_store_row(a, row, b, lane, acc, gated);
}

}  // namespace t3
