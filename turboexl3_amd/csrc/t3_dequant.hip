// W_hat: the trellis decoded to f16 [in][out], bit-exact to format.reconstructInner (turboexl3
// src/core/format.zig:276-291), and the test kernels that pin the reader and the codebooks on the device
// (the roles of turboexl3 src/kernels/hip/test/lane.hip's two kernels).

#include "t3_decode.hpp"
#include "t3_kernels.hpp"

namespace t3 {
namespace {

// Grid (ceil(out / 128 / kDqSteps), in / 16), 256 threads: a workgroup walks kDqSteps 128-column pieces of tile row tk; at
// every piece wave sg decodes tiles 8 piece + 2 sg and + 1, and the eight tiles' rows leave through LDS as 256-byte row
// segments, 16 bytes a thread. The lane plan is made once a workgroup, the next piece's words are fetched before the
// current piece is staged, and the stage alternates between two buffers: one barrier a piece.
constexpr uint32_t kDqSteps = 4u;
template <int CB, int WIDE>
__global__ void __launch_bounds__(256) dequant_kernel(const uint32_t* __restrict__ w, uint16_t* __restrict__ w_hat,
                                                      uint32_t out, uint32_t n, uint32_t wbits) {
    __shared__ __attribute__((aligned(16))) uint16_t stage[2][16][128 + 8];
    const uint32_t sg = threadIdx.x >> 6, lane = threadIdx.x & 63u;
    const uint32_t tk = blockIdx.y;
    const uint32_t out_tiles = out >> 4, nw = n >> 1;
    const QuadPlan<WIDE> plan = quad_plan<WIDE>(n, lane);
    const uint32_t* row = w + static_cast<size_t>(tk) * out_tiles * nw;
    const uint32_t first = blockIdx.x * kDqSteps;  // 128-column pieces
    // a tile past the row's last reads tile 0 again: decoded, staged and never stored
    auto fetch = [&](uint32_t piece, QuadWords<WIDE>(&wd)[2]) {
#pragma unroll
        for (uint32_t t = 0; t < 2u; ++t) {
            const uint32_t tn = piece * 8u + 2u * sg + t;
            wd[t] = quad_load<WIDE>(row + static_cast<size_t>(tn < out_tiles ? tn : 0u) * nw, plan);
        }
    };
    QuadWords<WIDE> cur[2], nxt[2];
    fetch(first, cur);
    const uint32_t r = threadIdx.x >> 4, c8 = (threadIdx.x & 15u) * 8u;
    for (uint32_t s = 0; s < kDqSteps; ++s) {
        const uint32_t piece = first + s;
        if (piece * 128u >= out) break;  // uniform over the workgroup
        if (s + 1u < kDqSteps) fetch(piece + 1u, nxt);
        uint16_t(*st)[128 + 8] = stage[s & 1u];
#pragma unroll
        for (uint32_t t = 0; t < 2u; ++t) {
            uint32_t cw[4];
            quad_codewords<WIDE>(cur[t], plan, wbits, cw);
#pragma unroll
            for (uint32_t m = 0; m < 4u; ++m)
                st[quad_row(lane, m)][(2u * sg + t) * 16u + quad_col(lane)] = decode_exact<CB>(cw[m]);
        }
        __syncthreads();
        const uint32_t col = piece * 128u + c8;
        if (col < out)  // out is a multiple of 64: a piece's second half may lie past the end
            *reinterpret_cast<uint4*>(w_hat + (static_cast<size_t>(tk) * 16u + r) * out + col) =
                *reinterpret_cast<const uint4*>(&st[r][c8]);
#pragma unroll
        for (uint32_t t = 0; t < 2u; ++t) cur[t] = nxt[t];
    }
}

__global__ void __launch_bounds__(256) test_codebooks_kernel(uint16_t* mcg, uint16_t* mul1, uint16_t* t) {
    const uint32_t cw = blockIdx.x * 256u + threadIdx.x;
    mcg[cw] = decode_mcg(cw);
    mul1[cw] = decode_mul1(cw);
    t[cw] = static_cast<uint16_t>(mul1_t(cw));
}

// Grid (tiles), 64 threads: the quad reader's codewords by code position and both codebooks' values of them.
template <int WIDE>
__global__ void __launch_bounds__(64) test_lane_kernel(const uint32_t* trellis, uint32_t n, uint32_t wbits,
                                                       uint16_t* cw_out, uint16_t* mcg, uint16_t* mul1) {
    const uint32_t lane = threadIdx.x, tile = blockIdx.x;
    const QuadPlan<WIDE> plan = quad_plan<WIDE>(n, lane);
    const QuadWords<WIDE> words = quad_load<WIDE>(trellis + static_cast<size_t>(tile) * (n >> 1), plan);
    uint32_t cw[4];
    quad_codewords<WIDE>(words, plan, wbits, cw);
    const uint32_t p = quad_first_position(lane);
#pragma unroll
    for (uint32_t m = 0; m < 4u; ++m) {
        const size_t at = static_cast<size_t>(tile) * 256u + p + m;
        cw_out[at] = static_cast<uint16_t>(cw[m]);
        mcg[at] = decode_mcg(cw[m]);
        mul1[at] = decode_mul1(cw[m]);
    }
}

// One wave: D [16][16] = A [16][32] B [32][16] (row-major f16 in, f32 out) with the GEMV's fragment assumptions:
// lane l supplies A[l % 16][8 (l / 16) .. + 7] and B[8 (l / 16) .. + 7][l % 16], and receives D[4 (l / 16) + r][l % 16].
__global__ void __launch_bounds__(64) test_mfma_kernel(const uint16_t* a, const uint16_t* b, float* d) {
    const uint32_t lane = threadIdx.x, i = lane & 15u, g = lane >> 4;
    half8 av, bv;
#pragma unroll
    for (uint32_t k = 0; k < 8u; ++k) {
        av[k] = __builtin_bit_cast(_Float16, a[i * 32u + 8u * g + k]);
        bv[k] = __builtin_bit_cast(_Float16, b[(8u * g + k) * 16u + i]);
    }
    float4v acc = {0.f, 0.f, 0.f, 0.f};
    acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(av, bv, acc, 0, 0, 0);
#pragma unroll
    for (uint32_t r = 0; r < 4u; ++r) d[(4u * g + r) * 16u + i] = acc[r];
}

}  // namespace

hipError_t launch_dequant(const uint32_t* trellis, uint16_t* w_hat, uint32_t in, uint32_t out, uint32_t n,
                          uint32_t wbits, int codebook, hipStream_t s) {
    const dim3 grid((out + 128u * kDqSteps - 1u) / (128u * kDqSteps), in / 16u), block(256);
    const bool mcg = codebook == kMcg || codebook == kMcgPair;
    with_reader(n, [&](auto reader) {
        constexpr int R = decltype(reader)::value;
        if (mcg) hipLaunchKernelGGL((dequant_kernel<kMcg, R>), grid, block, 0, s, trellis, w_hat, out, n, wbits);
        else hipLaunchKernelGGL((dequant_kernel<kMul1, R>), grid, block, 0, s, trellis, w_hat, out, n, wbits);
    });
    return hipGetLastError();
}

hipError_t launch_test_codebooks(uint16_t* mcg, uint16_t* mul1, uint16_t* t, hipStream_t s) {
    hipLaunchKernelGGL(test_codebooks_kernel, dim3(256), dim3(256), 0, s, mcg, mul1, t);
    return hipGetLastError();
}

hipError_t launch_test_lane(const uint32_t* trellis, uint32_t n, uint32_t wbits, uint32_t tiles, uint16_t* cw,
                            uint16_t* mcg, uint16_t* mul1, hipStream_t s) {
    with_reader(n, [&](auto reader) {
        hipLaunchKernelGGL(test_lane_kernel<decltype(reader)::value>, dim3(tiles), dim3(64), 0, s, trellis, n, wbits, cw,
                           mcg, mul1);
    });
    return hipGetLastError();
}

namespace {
// Grid (ceil(count / 256)), 256 threads: every value through the kernels' own narrowing and widening
__global__ void __launch_bounds__(256) test_convert_kernel(const float* in, uint16_t* bf16, uint16_t* f16, float* back,
                                                           uint32_t count) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i >= count) return;
    bf16[i] = bf16_bits(in[i]);
    f16[i] = half_bits(in[i]);
    back[i] = bf16_value(bf16[i]);
}
}  // namespace

hipError_t launch_test_convert(const float* in, uint16_t* bf16, uint16_t* f16, float* back, uint32_t count, hipStream_t s) {
    hipLaunchKernelGGL(test_convert_kernel, dim3((count + 255u) / 256u), dim3(256), 0, s, in, bf16, f16, back, count);
    return hipGetLastError();
}

hipError_t launch_test_mfma(const uint16_t* a, const uint16_t* b, float* d, hipStream_t s) {
    hipLaunchKernelGGL(test_mfma_kernel, dim3(1), dim3(64), 0, s, a, b, d);
    return hipGetLastError();
}

namespace {
// A plain read of `pieces` 16-byte pieces, one a lane a step, the steps of a workgroup 256 pieces apart and the
// workgroups interleaved (piece = (step * grid + workgroup) * 256 + thread): what the memory system gives a kernel that
// does nothing with its bytes but fold them. Every lane's fold is stored, so no load can be dropped. Grid (wgs), 256
// threads; eight loads in flight a lane.
__global__ void __launch_bounds__(256) test_hbm_read_kernel(const uint4v* src, uint64_t pieces, uint32_t* sink) {
    const uint64_t stride = static_cast<uint64_t>(gridDim.x) * 256u;
    uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
    uint4v acc = {0u, 0u, 0u, 0u};
    for (; i + 7u * stride < pieces; i += 8u * stride) {
        uint4v v[8];
#pragma unroll
        for (uint32_t j = 0; j < 8u; ++j) v[j] = src[i + j * stride];
#pragma unroll
        for (uint32_t j = 0; j < 8u; ++j) acc ^= v[j];
    }
    for (; i < pieces; i += stride) acc ^= src[i];
    sink[blockIdx.x * 256u + threadIdx.x] = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
}
}  // namespace

hipError_t launch_test_hbm_read(const void* src, uint64_t bytes, uint32_t* sink, uint32_t workgroups, hipStream_t s) {
    hipLaunchKernelGGL(test_hbm_read_kernel, dim3(workgroups), dim3(256), 0, s, static_cast<const uint4v*>(src), bytes / 16u,
                       sink);
    return hipGetLastError();
}

}  // namespace t3
