// The un-rotated weight of a dense EXL3 linear on gfx950: W_std [in][out] in the activation dtype,
//   W_std = act(((H' (W_hat H))[i, o] / 128) * suh[i] * svh[o]),
// one rounding, so that y = x W_std is one plain GEMM (turboexl3 src/core/dense.zig:1600-1676: pass 1 `unrotCols` = the
// unscaled +-1 H128 of every 128-column block of every row of W_hat into f32; pass 2 `unrotRows` = the H128 of every
// 128-row block of every column, / 128, the two scale vectors, the rounding). Made once a weight; the per-call chain
// (prepare, trellis GEMM, finish) and its f16 roundings of x's rotated copy, of z and of the finish are not taken:
// the same linear map with other roundings (dense.zig:1597-1600).

#include "t3_kernels.hpp"
#include "t3_stages.hpp"

namespace t3 {
namespace {

// pass 1. One wave takes four adjacent 128-column blocks of one row of W_hat (16 lanes a block, 8 columns a lane).
// Grid ceil(rows * ceil(out / 512) / 4), 256 threads.
__global__ void __launch_bounds__(256) unrot_cols(const uint16_t* w_hat, float* r, uint32_t in, uint32_t out) {
    const uint32_t nb = out / 128u, groups = (nb + 3u) / 4u;
    const uint32_t u0 = blockIdx.x * 4u + (threadIdx.x >> 6), row = u0 / groups, lane = threadIdx.x & 63u;
    if (row >= in) return;
    const uint32_t b1 = (u0 % groups) * 4u + (lane >> 4);
    const bool live = b1 < nb;
    const uint32_t b = live ? b1 : nb - 1u;
    const size_t at = static_cast<size_t>(row) * out + b * 128u + 8u * (lane & 15u);
    const Row16 g = row16(lane);
    float v[8];
    load8_half(w_hat, at, v);
    h128_row16(v, g);
    const float sign = g.s1 * g.s2 * g.s4 * g.s8;  // the lane stages' deferred sign (t3_stages.hpp)
#pragma unroll
    for (uint32_t k = 0; k < 8u; ++k) v[k] *= sign;
    if (!live) return;
    *reinterpret_cast<float4v*>(r + at) = float4v{v[0], v[1], v[2], v[3]};
    *reinterpret_cast<float4v*>(r + at + 4) = float4v{v[4], v[5], v[6], v[7]};
}

// pass 2. One workgroup takes a 128-row block and a strip of 32 columns through LDS (33-float rows: a column's reads go
// to distinct banks); wave w transforms columns 8 w .. + 7, four at a time, 16 lanes a column and 8 rows a lane.
// Grid (out / 32, in / 128), 256 threads. nonfinite (may be null): counts the weights that left the dtype's range.
template <int DT>
__global__ void __launch_bounds__(256) unrot_rows(const float* r, const uint16_t* suh, const uint16_t* svh, void* w_std,
                                                  uint32_t out, uint32_t ld, uint32_t col0, uint32_t* nonfinite) {
    __shared__ float tile[128][33];
    const uint32_t c0 = blockIdx.x * 32u, r0 = blockIdx.y * 128u;
    const uint32_t wave = threadIdx.x >> 6, lane = threadIdx.x & 63u, q = lane & 15u;
    for (uint32_t i = threadIdx.x; i < 128u * 32u; i += 256u)
        tile[i >> 5][i & 31u] = r[static_cast<size_t>(r0 + (i >> 5)) * out + c0 + (i & 31u)];
    __syncthreads();
    const Row16 g = row16(lane);
    uint32_t bad = 0;
#pragma unroll
    for (uint32_t pass = 0; pass < 2u; ++pass) {
        const uint32_t c = wave * 8u + pass * 4u + (lane >> 4);
        float v[8];
#pragma unroll
        for (uint32_t k = 0; k < 8u; ++k) v[k] = tile[8u * q + k][c];
        h128_row16(v, g);
        const float sign = g.s1 * g.s2 * g.s4 * g.s8;
        const float sv = half_value(svh[c0 + c]);
#pragma unroll
        for (uint32_t k = 0; k < 8u; ++k) {
            const float w = ((v[k] * sign) * (1.0f / 128.0f)) * half_value(suh[r0 + 8u * q + k]) * sv;
            float rounded;
            if constexpr (DT == kF16) rounded = round_half(w);
            else rounded = bf16_value(bf16_bits(w));
            bad += (rounded - rounded != 0.0f) ? 1u : 0u;  // an infinity or a NaN
            tile[8u * q + k][c] = rounded;
        }
    }
    __syncthreads();
    for (uint32_t i = threadIdx.x; i < 128u * 32u; i += 256u)
        store_act<DT>(w_std, static_cast<size_t>(r0 + (i >> 5)) * ld + col0 + c0 + (i & 31u), tile[i >> 5][i & 31u]);
    if (nonfinite && bad) atomicAdd(nonfinite, bad);
}

}  // namespace

hipError_t launch_unrot(const uint16_t* w_hat, float* r, const uint16_t* suh, const uint16_t* svh, void* w_std, uint32_t in,
                        uint32_t out, uint32_t ld, uint32_t col0, int dtype, uint32_t* nonfinite, hipStream_t s) {
    const uint32_t groups = (out / 128u + 3u) / 4u;
    hipLaunchKernelGGL(unrot_cols, dim3((in * groups + 3u) / 4u), dim3(256), 0, s, w_hat, r, in, out);
    if (const hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    const dim3 grid(out / 32u, in / 128u);
    if (dtype == kF16) hipLaunchKernelGGL(unrot_rows<kF16>, grid, dim3(256), 0, s, r, suh, svh, w_std, out, ld, col0, nonfinite);
    else hipLaunchKernelGGL(unrot_rows<kBf16>, grid, dim3(256), 0, s, r, suh, svh, w_std, out, ld, col0, nonfinite);
    return hipGetLastError();
}

}  // namespace t3
