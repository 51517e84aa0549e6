// Dense EXL3 projection at decode rows (1..32) on gfx950: prepare -> trellis GEMV on the matrix cores -> finish.
//
// The chain computes format.project's stages (turboexl3 src/core/format.zig:334-389) with its rounding points:
//   prepare  xp = f16(H128(f16(x) * suh) / sqrt(128)) per 128-block, stored in quad order with every value doubled
//            (the B fragment of the GEMV's MFMA), plus each block's sum of xp (the deferred MUL1 map's input);
//   gemv     z[slice] = xp * W_hat over one K slice: each wave decodes one 16x16 tile at a time, a quad of weights a
//            lane, straight into the A fragment of v_mfma_f32_16x16x32_f16; no decoded weight is written anywhere;
//   finish   planes summed in slice order -> (deferred map) -> f16 -> H128 -> * svh / sqrt(128) -> f16 -> y's dtype.
// The K partition (slices x 4 waves) depends on (in, out) alone, and every output element of the MFMA depends on its
// own row of x alone, so a row's bytes do not depend on the rows beside it (the reference's row-alone invariant,
// turboexl3 src/hip_tests.zig:338-346).
//
// The role of each launch follows the reference's HIP plan (src/hip/plan.zig:161-204) but the launch shapes, the lane
// plan and the use of MFMA are this library's own.

#include "t3_decode.hpp"
#include "t3_kernels.hpp"

namespace t3 {
namespace {

// Grid (in / 128, rows), 64 threads. xq: uint32 [rows][in], word (tk 16 + quad_slot(r)) = the f16 value of input
// tk 16 + r in both halves. xs: f32 [rows][in / 128].
template <int DT>
__device__ __forceinline__ void prep_block(const void* x, const uint16_t* suh, uint32_t* xq, float* xs, uint32_t in,
                                           uint32_t row_in, uint32_t row_out, uint32_t b, uint32_t lane) {
    float v[2];
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
        const uint32_t i = b * 128u + lane + 64u * j;
        v[j] = round_half(load_act<DT>(x, static_cast<size_t>(row_in) * in + i)) * half_value(suh[i]);
    }
    h128_wave(v, lane);
    float sum = 0.0f;
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
        const uint32_t i = b * 128u + lane + 64u * j;
        const uint32_t hv = half_bits(v[j] * kHadScale);
        xq[static_cast<size_t>(row_out) * in + (i & ~15u) + quad_slot(i & 15u)] = hv | (hv << 16);
        sum += half_value(hv);
    }
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) sum += __shfl_xor(sum, m, 64);
    if (lane == 0u) xs[static_cast<size_t>(row_out) * (in / 128u) + b] = sum;
}

template <int DT>
__global__ void __launch_bounds__(64) dense_prep(const void* x, const uint16_t* suh, uint32_t* xq, float* xs,
                                                 uint32_t in) {
    prep_block<DT>(x, suh, xq, xs, in, blockIdx.y, blockIdx.y, blockIdx.x, threadIdx.x);
}

// Grid (out / 16 / BT, KS), 256 threads (4 waves). A workgroup owns BT adjacent output tiles and K slice blockIdx.y;
// wave sg takes part sg of the slice, `per` = in_tiles / (4 KS) input tiles (the host divides: the GPU has no scalar divide). RB = 16-row blocks of x (1 or 2).
// z f32 [KS][rows][out]: the four waves' sums, wave 0 first.
template <int CB, bool WIDE, int RB, int BT>
__global__ void __launch_bounds__(256) dense_gemv(const uint32_t* __restrict__ w, const uint32_t* __restrict__ xq,
                                                  float* __restrict__ z, uint32_t in, uint32_t out, uint32_t rows,
                                                  uint32_t n, uint32_t wbits, uint32_t per) {
    __shared__ float4v red[4][RB * BT * 64];
    const uint32_t blk = blockIdx.x, ksl = blockIdx.y;
    const uint32_t sg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63u;
    const uint32_t in_tiles = in >> 4, out_tiles = out >> 4, nw = n >> 1;
    const uint32_t tk0 = (ksl * 4u + sg) * per;
    const QuadPlan<WIDE> plan = quad_plan<WIDE>(n, lane);

    float4v acc[RB][BT];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int t = 0; t < BT; ++t) acc[r][t] = float4v{0.f, 0.f, 0.f, 0.f};

    // x fragment: activation row (lane % 16) of block r, K slots 8g..8g+7 = quad g's four inputs, each doubled.
    // Rows past the call's last alias row 0: their sums are computed and never stored.
    const uint32_t g = lane >> 4;
    uint32_t xoff[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) {
        const uint32_t row = static_cast<uint32_t>(r) * 16u + (lane & 15u);
        xoff[r] = ((row < rows ? row : 0u) * in + 4u * g) * 4u;
    }
    // Per-lane byte offsets inside the workgroup's BT adjacent tiles; the tile row's offset stays scalar.
    uint32_t off_bp[BT], off_bl[BT], off_ap[BT], off_al[BT];
#pragma unroll
    for (int t = 0; t < BT; ++t) {
        off_bp[t] = (static_cast<uint32_t>(t) * nw + plan.ib_prev) * 4u;
        off_bl[t] = (static_cast<uint32_t>(t) * nw + plan.ib_last) * 4u;
        off_ap[t] = (static_cast<uint32_t>(t) * nw + plan.ia_prev) * 4u;
        off_al[t] = (static_cast<uint32_t>(t) * nw + plan.ia_last) * 4u;
    }
    const uint64_t wstride = static_cast<uint64_t>(out_tiles) * nw;  // words a tile row
    const uint64_t wfirst = static_cast<uint64_t>(blk) * BT * nw + tk0 * wstride;
    const __amdgpu_buffer_rsrc_t wres = make_rsrc(w + wfirst, (static_cast<uint64_t>(in_tiles) * wstride - wfirst) * 4u);
    const __amdgpu_buffer_rsrc_t xres = make_rsrc(xq, static_cast<uint64_t>(rows) * in * 4u);
    const uint32_t wstep = static_cast<uint32_t>(wstride) * 4u;  // bytes; the host holds a matrix under 2^31 bytes
    const uint32_t wstep2 = 2u * wstep;

    auto load_tiles = [&](uint32_t soff, QuadWords<WIDE>(&dst)[BT]) {
#pragma unroll
        for (int t = 0; t < BT; ++t) {
            dst[t].b_prev = buf_load_u32(wres, off_bp[t], soff);
            dst[t].b_last = buf_load_u32(wres, off_bl[t], soff);
            if constexpr (WIDE) {
                dst[t].a_prev = buf_load_u32(wres, off_ap[t], soff);
                dst[t].a_last = buf_load_u32(wres, off_al[t], soff);
            }
        }
    };
    auto load_x = [&](uint32_t soff, uint4v(&dst)[RB]) {
#pragma unroll
        for (int r = 0; r < RB; ++r) dst[r] = buf_load_u128(xres, xoff[r], soff);
    };

    auto consume = [&](const QuadWords<WIDE>(&words)[BT], const uint4v(&xv)[RB]) {
#pragma unroll
        for (int t = 0; t < BT; ++t) {
            uint32_t cw[4];
            quad_codewords<WIDE>(words[t], plan, wbits, cw);
            uint4v a;
#pragma unroll
            for (int m = 0; m < 4; ++m) a[m] = weight_pair<CB>(cw[m]);
#pragma unroll
            for (int r = 0; r < RB; ++r)
                acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a),
                                                                   __builtin_bit_cast(half8, xv[r]), acc[r][t], 0, 0, 0);
        }
    };

    // Two register sets in turn: while one tile row decodes, the next one's words are in flight.
    QuadWords<WIDE> wa[BT], wb[BT];
    uint4v xa[RB], xb[RB];
    uint32_t wo = 0u, xo = tk0 * 64u;  // scalar byte offsets of the tile row in flight
    load_tiles(wo, wa);
    load_x(xo, xa);
    uint32_t i = 0;
    for (; i + 1u < per; i += 2u) {
        load_tiles(wo + wstep, wb);
        load_x(xo + 64u, xb);
        __builtin_amdgcn_sched_barrier(0);
        consume(wa, xa);
        const bool two = i + 2u < per;  // the last odd step rereads the row already held
        wo += two ? wstep2 : wstep;
        xo += two ? 128u : 64u;
        load_tiles(wo, wa);
        load_x(xo, xa);
        __builtin_amdgcn_sched_barrier(0);
        consume(wb, xb);
    }
    if (i < per) consume(wa, xa);

    // lane holds, for activation row (lane % 16) of block r, output columns 4g..4g+3 of tile t
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int t = 0; t < BT; ++t) red[sg][(r * BT + t) * 64 + lane] = acc[r][t];
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < static_cast<uint32_t>(RB * BT * 64); i += 256u) {
        const uint32_t l = i & 63u, t = (i >> 6) % BT, r = (i >> 6) / BT;
        const uint32_t row = r * 16u + (l & 15u);
        if (row >= rows) continue;
        const float4v s = ((red[0][i] + red[1][i]) + red[2][i]) + red[3][i];
        float* dst = z + (static_cast<size_t>(ksl) * rows + row) * out + (blk * BT + t) * 16u + 4u * (l >> 4);
        *reinterpret_cast<float4v*>(dst) = s;
    }
}

// Grid (out / 128, rows), 64 threads: lane L finishes outputs b 128 + L and + 64.
template <int DT>
__device__ __forceinline__ void finish_block(const float* z, const float* xs, const uint16_t* svh, void* y,
                                             uint32_t out, uint32_t rows, uint32_t ks, uint32_t inblk, int defer,
                                             uint32_t row, uint32_t b, uint32_t lane) {
    float xsum = 0.0f;
    if (defer)
        for (uint32_t q = 0; q < inblk; ++q) xsum += xs[static_cast<size_t>(row) * inblk + q];
    float v[2];
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
        const uint32_t o = b * 128u + lane + 64u * j;
        float acc = z[static_cast<size_t>(row) * out + o];
        for (uint32_t k = 1u; k < ks; ++k) acc += z[(static_cast<size_t>(k) * rows + row) * out + o];
        if (defer) acc = __builtin_fmaf(acc, mul1_a(), mul1_b() * xsum);
        v[j] = round_half(acc);
    }
    h128_wave(v, lane);
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
        const uint32_t o = b * 128u + lane + 64u * j;
        store_act<DT>(y, static_cast<size_t>(row) * out + o, round_half(v[j] * kHadScale * half_value(svh[o])));
    }
}

template <int DT>
__global__ void __launch_bounds__(64) dense_finish(const float* z, const float* xs, const uint16_t* svh, void* y,
                                                   uint32_t out, uint32_t rows, uint32_t ks, uint32_t inblk,
                                                   int defer) {
    finish_block<DT>(z, xs, svh, y, out, rows, ks, inblk, defer, blockIdx.y, blockIdx.x, threadIdx.x);
}

template <int CB, bool WIDE, int RB>
hipError_t launch_gemv_bt(const DenseLaunch& d, hipStream_t s) {
    const dim3 block(256);
    const uint32_t out_tiles = d.out / 16u;
    auto go = [&](auto kern, uint32_t bt) {
        hipLaunchKernelGGL(kern, dim3(out_tiles / bt, d.ks), block, 0, s, d.trellis, d.xq, d.z, d.in, d.out, d.rows,
                           d.n, d.wbits, (d.in / 16u) / (4u * d.ks));
        return hipGetLastError();
    };
    switch (d.bt) {
        case 1: return go(dense_gemv<CB, WIDE, RB, 1>, 1u);
        case 2: return go(dense_gemv<CB, WIDE, RB, 2>, 2u);
        default: return go(dense_gemv<CB, WIDE, RB, 4>, 4u);
    }
}

template <int CB>
hipError_t launch_gemv_cb(const DenseLaunch& d, hipStream_t s) {
    const bool wide = quad_needs_wide(d.n);
    const bool two = d.rows > 16u;
    if (wide) return two ? launch_gemv_bt<CB, true, 2>(d, s) : launch_gemv_bt<CB, true, 1>(d, s);
    return two ? launch_gemv_bt<CB, false, 2>(d, s) : launch_gemv_bt<CB, false, 1>(d, s);
}

}  // namespace

hipError_t launch_dense_prep(const DenseLaunch& d, hipStream_t s) {
    const dim3 grid(d.in / 128u, d.rows), block(64);
    switch (d.dtype) {
        case kF32: hipLaunchKernelGGL(dense_prep<kF32>, grid, block, 0, s, d.x, d.suh, d.xq, d.xs, d.in); break;
        case kF16: hipLaunchKernelGGL(dense_prep<kF16>, grid, block, 0, s, d.x, d.suh, d.xq, d.xs, d.in); break;
        default: hipLaunchKernelGGL(dense_prep<kBf16>, grid, block, 0, s, d.x, d.suh, d.xq, d.xs, d.in); break;
    }
    return hipGetLastError();
}

hipError_t launch_dense_gemv(const DenseLaunch& d, hipStream_t s) {
    switch (d.codebook) {
        case kMul1: return launch_gemv_cb<kMul1>(d, s);
        case kMcg: return launch_gemv_cb<kMcg>(d, s);
        case kMul1Defer: return launch_gemv_cb<kMul1Defer>(d, s);
        default: return launch_gemv_cb<kMcgPair>(d, s);
    }
}

hipError_t launch_dense_finish(const DenseLaunch& d, hipStream_t s) {
    const dim3 grid(d.out / 128u, d.rows), block(64);
    const int defer = d.codebook == kMul1Defer;
    const uint32_t inblk = d.in / 128u;
    switch (d.dtype) {
        case kF32:
            hipLaunchKernelGGL(dense_finish<kF32>, grid, block, 0, s, d.z, d.xs, d.svh, d.y, d.out, d.rows, d.ks, inblk,
                               defer);
            break;
        case kF16:
            hipLaunchKernelGGL(dense_finish<kF16>, grid, block, 0, s, d.z, d.xs, d.svh, d.y, d.out, d.rows, d.ks, inblk,
                               defer);
            break;
        default:
            hipLaunchKernelGGL(dense_finish<kBf16>, grid, block, 0, s, d.z, d.xs, d.svh, d.y, d.out, d.rows, d.ks, inblk,
                               defer);
            break;
    }
    return hipGetLastError();
}

}  // namespace t3
