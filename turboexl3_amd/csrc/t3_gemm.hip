// The plain half-precision GEMM of the dense paths above 32 rows on gfx950: y [rows][cols] = x [rows][in] w [in][ldw],
// f16 or bf16 operands, f32 accumulation on the matrix cores, one rounding at the store. It multiplies a decoded W_hat
// (the reference's dequant + matmul + finish form, turboexl3 src/core/dense.zig:909-922,1290-1302, where the product is
// MLX's matmul; its HIP backend runs its own matrix-unit GEMM there, src/hip/plan.zig:478-495) and the un-rotated
// resident weight W_std (src/core/dense.zig:1612-1690).
//
// Shape. A workgroup of eight waves takes 256 rows x 256 columns; wave (wm, wn) of the 2 x 4 grid owns 128 rows x 64
// columns: 8 x 4 blocks of v_mfma_f32_16x16x32 with the WEIGHTS as the A operand (M = 16 output columns) and the
// activations as B (N = 16 rows), so a lane ends with four adjacent output columns of one row. K advances 32 a step.
//
// Memory path. Both operands go from memory straight into LDS (buffer_load ... lds: lane L's 16 bytes land at
// M0 + 16 L), four steps deep, 32 KB a step; the kernel counts those loads itself (s_waitcnt vmcnt(N)) and issues no
// other vector-memory load while they fly. Which global piece a lane fetches decides the LDS layout at 16-byte
// granularity, so both tiles are swizzled for their readers on the way in, at no cost:
//   activations  [256 rows][32 k], 64 bytes a row; the 16-byte piece p of row r sits at position p ^ ((r >> 1) & 3):
//                a B fragment (16 rows x one piece) then spreads over all banks (ds_read_b128);
//   weights      [32 k][256 columns] as they lie in memory (k-major), 512 bytes a row; piece s of row k sits at
//                position s ^ f(k), f(k) = 2 ((k & 3) + 4 ((k >> 3) & 1)). The A fragment wants eight consecutive k of
//                ONE column a lane, which a k-major tile holds 512 bytes apart: gfx950's transposing LDS read
//                (ds_read_b64_tr_b16: inside every 16 lanes, the 4 x 16 halfwords the lanes address are transposed, lane
//                i receiving column i) delivers them, two reads a fragment, and f(k) spreads one such read's sixteen
//                rows over the banks.
// Workgroup ids: consecutive ids go round the eight dies; a die takes column blocks nt = 8 j + die and walks every row
// block of one column block before the next, so a die's L2 holds the weight strip its workgroups share.

#include "t3_common.hpp"
#include "t3_kernels.hpp"

namespace t3 {
namespace {

constexpr uint32_t kGM = 256, kGN = 256, kGK = 32, kGD = 4;     // tile rows, columns, K a step, steps in the ring
constexpr uint32_t kGXBytes = kGM * kGK * 2u, kGWBytes = kGK * kGN * 2u, kGStep = kGXBytes + kGWBytes;
constexpr int kGLoadsAStep = 4;                                  // loads a wave a step: two of x, two of w

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) short4v lds_short4v;

struct GemmArgs {
    const void* x;
    const void* w;
    void* y;
    uint32_t rows, in, cols, ldw, mt, nt;
};

__device__ __forceinline__ uint4v gemm_rsrc(const void* p, uint64_t bytes) {
    const uint64_t addr = reinterpret_cast<uint64_t>(p);
    const uint32_t n = bytes > 0xFFFFFFFFull ? 0xFFFFFFFFu : static_cast<uint32_t>(bytes);
    return uint4v{static_cast<uint32_t>(addr), static_cast<uint32_t>(addr >> 32) & 0xFFFFu, n, 0x00020000u};
}
__device__ __forceinline__ void gemm_load_to_lds(uint4v desc, uint32_t lds, uint32_t voff, uint32_t soff) {
    asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tbuffer_load_dwordx4 %1, %2, %3 offen lds"
                 :
                 : "s"(lds), "v"(voff), "s"(desc), "s"(soff)
                 : "memory");
}
template <int N>
__device__ __forceinline__ void gemm_wait_loads() {
    asm volatile("s_waitcnt vmcnt(%0)" : : "n"(N) : "memory");
}

template <bool BF16>
__device__ __forceinline__ float4v gemm_mfma(uint4v a, uint4v b, float4v c) {
    if constexpr (BF16)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), c, 0, 0, 0);
}

// Grid (8 mt, ceil(nt / 8)), 512 threads.
template <bool BF16>
__global__ void __launch_bounds__(512) gemm_half(const GemmArgs a) {
    __shared__ __attribute__((aligned(16))) unsigned char smem[kGD * kGStep];
    const uint32_t die = blockIdx.x & 7u, mi = blockIdx.x >> 3, ni = blockIdx.y * 8u + die;
    if (ni >= a.nt) return;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63u;
    const uint32_t wm = wave & 1u, wn = wave >> 1;
    const uint32_t row0 = mi * kGM, col0 = ni * kGN;

    // the tile's windows of x and w: rows past the last one, and the bytes past w's end, read as zeros
    const uint32_t rows_here = a.rows - row0 < kGM ? a.rows - row0 : kGM;
    const uint4v xdesc = gemm_rsrc(static_cast<const unsigned char*>(a.x) + static_cast<size_t>(row0) * a.in * 2u,
                                   static_cast<uint64_t>(rows_here) * a.in * 2u);
    const uint4v wdesc = gemm_rsrc(static_cast<const unsigned char*>(a.w) + static_cast<size_t>(col0) * 2u,
                                   (static_cast<uint64_t>(a.in) * a.ldw - col0) * 2u);
    // this wave's loads a step: x rows 32 wave .. + 31 (two loads of 16 rows), w rows k = 4 wave .. + 3 (two of 2 rows)
    uint32_t x_voff[2], w_voff[2];
#pragma unroll
    for (uint32_t i = 0; i < 2u; ++i) {
        const uint32_t row = (2u * wave + i) * 16u + (lane >> 2), piece = (lane & 3u) ^ ((lane >> 3) & 3u);
        x_voff[i] = row < rows_here ? (row * a.in + piece * 8u) * 2u : 0x80000000u;
        const uint32_t k = (2u * wave + i) * 2u + (lane >> 5);
        const uint32_t fk = 2u * ((k & 3u) + 4u * ((k >> 3) & 1u));
        w_voff[i] = (k * a.ldw + ((lane & 31u) ^ fk) * 8u) * 2u;
    }
    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem));
    const uint32_t w_step_bytes = kGK * a.ldw * 2u;
    auto issue = [&](uint32_t step, uint32_t slot) {
        const uint32_t base = lds0 + slot * kGStep;
#pragma unroll
        for (uint32_t i = 0; i < 2u; ++i) gemm_load_to_lds(xdesc, base + (2u * wave + i) * 1024u, x_voff[i], step * (kGK * 2u));
#pragma unroll
        for (uint32_t i = 0; i < 2u; ++i)
            gemm_load_to_lds(wdesc, base + kGXBytes + (2u * wave + i) * 1024u, w_voff[i], step * w_step_bytes);
    };

    // where a lane's fragments sit inside a step's 32 KB
    // activations, row block rb: row 128 wm + 16 rb + lane % 16, piece lane / 16, swizzled
    const uint32_t xf_at = (128u * wm + (lane & 15u)) * 64u + (((lane >> 4) ^ ((lane >> 1) & 3u)) * 16u);
    // weights, column block cb, half h: row k = 8 g + 4 h + j / 4, columns 16 (4 wn + cb) + 4 (j % 4) .. + 3
    const uint32_t g = lane >> 4, j = lane & 15u;
    const uint32_t fk = 2u * ((j >> 2) + 4u * (g & 1u));
    uint32_t wf_at[4];
#pragma unroll
    for (uint32_t cb = 0; cb < 4u; ++cb) {
        const uint32_t piece = (8u * wn + 2u * cb + ((j >> 1) & 1u)) ^ fk;
        wf_at[cb] = kGXBytes + (8u * g + (j >> 2)) * 512u + piece * 16u + (j & 1u) * 8u;
    }

    float4v acc[4][8];
#pragma unroll
    for (int cb = 0; cb < 4; ++cb)
#pragma unroll
        for (int rb = 0; rb < 8; ++rb) acc[cb][rb] = float4v{0.f, 0.f, 0.f, 0.f};

    const uint32_t steps = a.in / kGK;
#pragma unroll
    for (uint32_t t = 0; t + 1u < kGD; ++t) issue(t, t);   // loads past the last step fall outside the buffers: zeros
    gemm_wait_loads<static_cast<int>(kGD - 2u) * kGLoadsAStep>();
    __syncthreads();
    uint32_t slot = 0;
    for (uint32_t s = 0; s < steps; ++s) {
        // the slot step s - 1 used is free: every wave passed the barrier that ended it
        issue(s + kGD - 1u, slot == 0u ? kGD - 1u : slot - 1u);
        const unsigned char* st = smem + slot * kGStep;
        uint4v wf[4], xf[8];
#pragma unroll
        for (uint32_t cb = 0; cb < 4u; ++cb) {
            const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4v*)(st + wf_at[cb]));
            const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4v*)(st + wf_at[cb] + 4u * 512u));
            const uint2 l2 = __builtin_bit_cast(uint2, lo), h2 = __builtin_bit_cast(uint2, hi);
            wf[cb] = uint4v{l2.x, l2.y, h2.x, h2.y};
        }
#pragma unroll
        for (uint32_t rb = 0; rb < 8u; ++rb) xf[rb] = *reinterpret_cast<const uint4v*>(st + xf_at + rb * 1024u);
#pragma unroll
        for (int cb = 0; cb < 4; ++cb)
#pragma unroll
            for (int rb = 0; rb < 8; ++rb) acc[cb][rb] = gemm_mfma<BF16>(wf[cb], xf[rb], acc[cb][rb]);
        // step s + 1's loads of this wave have landed once at most kGD - 2 steps' are in flight; the barrier then
        // publishes every wave's part of it
        gemm_wait_loads<static_cast<int>(kGD - 2u) * kGLoadsAStep>();
        __syncthreads();
        slot = slot + 1u == kGD ? 0u : slot + 1u;
    }
    gemm_wait_loads<0>();

    // lane: row 16 rb + lane % 16, columns 16 cb + 4 (lane / 16) .. + 3 of the wave's 128 x 64
    const bool vec = (a.cols & 3u) == 0u;
#pragma unroll
    for (int rb = 0; rb < 8; ++rb) {
        const uint32_t row = row0 + 128u * wm + static_cast<uint32_t>(rb) * 16u + (lane & 15u);
        if (row >= a.rows) continue;
#pragma unroll
        for (int cb = 0; cb < 4; ++cb) {
            const uint32_t col = col0 + 64u * wn + static_cast<uint32_t>(cb) * 16u + 4u * (lane >> 4);
            if (col >= a.cols) continue;
            uint16_t h[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) h[c] = BF16 ? bf16_bits(acc[cb][rb][c]) : half_bits(acc[cb][rb][c]);
            uint16_t* dst = static_cast<uint16_t*>(a.y) + static_cast<size_t>(row) * a.cols + col;
            if (vec) {
                *reinterpret_cast<uint2*>(dst) = uint2{h[0] | (static_cast<uint32_t>(h[1]) << 16),
                                                       h[2] | (static_cast<uint32_t>(h[3]) << 16)};
            } else {
#pragma unroll
                for (uint32_t c = 0; c < 4u; ++c)
                    if (col + c < a.cols) dst[c] = h[c];
            }
        }
    }
}

}  // namespace

// y [rows][cols] = x [rows][in] w[:, 0:cols] for w [in][ldw] (all f16 or all bf16; y row-contiguous). The host has
// checked: in a multiple of 32, ldw a multiple of 8, w and x 16-byte aligned, in ldw 2 bytes under 4 GiB.
hipError_t launch_gemm_half(const void* x, const void* w, void* y, uint32_t rows, uint32_t in, uint32_t cols, uint32_t ldw,
                            bool bf16, hipStream_t s) {
    GemmArgs a;
    a.x = x;
    a.w = w;
    a.y = y;
    a.rows = rows;
    a.in = in;
    a.cols = cols;
    a.ldw = ldw;
    a.mt = (rows + kGM - 1u) / kGM;
    a.nt = (cols + kGN - 1u) / kGN;
    const dim3 grid(8u * a.mt, (a.nt + 7u) / 8u), block(512);
    if (bf16) hipLaunchKernelGGL(gemm_half<true>, grid, block, 0, s, a);
    else hipLaunchKernelGGL(gemm_half<false>, grid, block, 0, s, a);
    return hipGetLastError();
}

}  // namespace t3
