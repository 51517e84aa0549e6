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

#include "t3_gemv_core.hpp"
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
// wave sg takes part sg of the slice, `per` = in_tiles / (4 KS) input tiles (the host divides: the GPU has no scalar
// divide). RB = 16-row blocks of x (1 or 2). z f32 [KS][rows][out]: the four waves' sums, wave 0 first.
template <int CB, bool WIDE, int RB, int BT>
__global__ void __launch_bounds__(256) dense_gemv(const uint32_t* __restrict__ w, const uint32_t* __restrict__ xq,
                                                  float* __restrict__ z, uint32_t in, uint32_t out, uint32_t rows,
                                                  uint32_t n, uint32_t wbits, uint32_t per) {
    constexpr int ST = 8;  // tile rows in flight a wave
    constexpr uint32_t kStage = gemv_stage_bytes<BT>();
    constexpr uint32_t kRed = 4u * RB * BT * 64u * 16u;
    // the waves' LDS stages while they stream; the four waves' partial sums afterwards
    __shared__ __attribute__((aligned(16))) unsigned char smem[kRed > 4u * kStage ? kRed : 4u * kStage];
    float4v(*red)[RB * BT * 64] = reinterpret_cast<float4v(*)[RB * BT * 64]>(smem);
    const uint32_t blk = blockIdx.x, ksl = blockIdx.y;
    const uint32_t sg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63u;
    const uint32_t out_tiles = out >> 4, nw = n >> 1;
    const uint32_t tk0 = (ksl * 4u + sg) * per;
    const QuadPlan<WIDE> plan = quad_plan<WIDE>(n, lane);

    float4v acc[RB][BT];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int t = 0; t < BT; ++t) acc[r][t] = float4v{0.f, 0.f, 0.f, 0.f};

    // x fragment: activation row (lane % 16) of block r, K slots 8g..8g+7 = quad g's four inputs, each doubled.
    // Rows past the call's last alias row 0: their sums are computed and never stored.
    uint32_t xoff[RB];
#pragma unroll
    for (int r = 0; r < RB; ++r) {
        const uint32_t row = static_cast<uint32_t>(r) * 16u + (lane & 15u);
        xoff[r] = ((row < rows ? row : 0u) * in + 4u * (lane >> 4)) * 4u;
    }
    const uint64_t wstride = static_cast<uint64_t>(out_tiles) * nw;  // words a tile row
    const uint32_t* wbase = w + static_cast<uint64_t>(blk) * BT * nw + tk0 * wstride;
    gemv_stream<CB, WIDE, RB, BT, ST>(wbase, static_cast<uint32_t>(wstride) * 4u, per, n, plan, wbits, xq,
                                      static_cast<uint64_t>(rows) * in * 4u, xoff, tk0 * 64u, smem + sg * kStage, lane,
                                      acc);
    __syncthreads();  // every wave is done with its stage before the sums take the memory

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
    if (d.bt == 8u) return go(dense_gemv<CB, WIDE, RB, 8>, 8u);
    return go(dense_gemv<CB, WIDE, RB, 4>, 4u);
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
