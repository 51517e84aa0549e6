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
// The end. The accumulators go to LDS as one 256 x 256 tile of halfwords (528-byte rows, so the matrix-core layout's
// 16 rows a store spread over the banks), and leave it 16 bytes a lane, 256 contiguous bytes a row segment. FINISH: the
// tile is z = f16(xp W_hat), format.innerGemv's rounding point (src/core/format.zig:366), and the launch ends with
// format.finishOutput (:370-380) on it: four 128-blocks a wave, 16 lanes a block, the statements of the prefill chains'
// finish kernel, then y in the call's dtype. z never sees memory.
// Workgroup ids: consecutive ids go round the eight dies; a die takes column blocks nt = 8 j + die and walks every row
// block of one column block before the next, so a die's L2 holds the weight strip its workgroups share. A workgroup
// holds a compute unit alone (135 KB of LDS), so the launch runs in rounds of 256 workgroups; where the last round would
// fill at most half the GPU, its column blocks are cut to 128 columns (the same kernel with two column blocks a wave):
// 4096 rows x 14336 columns is 896 tiles = 3.5 rounds, and runs as 768 full tiles + 256 half ones.

#include "t3_common.hpp"
#include "t3_kernels.hpp"
#include "t3_lds_loads.hpp"
#include "t3_stages.hpp"

namespace t3 {
namespace {

constexpr uint32_t kGM = 256, kGN = 256, kGK = 32, kGD = 4;     // tile rows, columns, K a step, steps in the ring
constexpr uint32_t kGXBytes = kGM * kGK * 2u, kGWBytes = kGK * kGN * 2u, kGStep = kGXBytes + kGWBytes;
constexpr int kGLoadsAStep = 4;                                  // loads a wave a step: two of x, two of w
constexpr uint32_t kGZRow = kGN * 2u + 16u;                      // bytes a row of the output tile in LDS
constexpr uint32_t kGLds = kGD * kGStep > kGM * kGZRow ? kGD * kGStep : kGM * kGZRow;

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) short4v lds_short4v;

struct GemmArgs {
    const void* x;
    const void* w;
    void* y;
    const uint16_t* svh;  // FINISH: the output scale vector f16 [cols]
    int dt;               // FINISH: y's dtype (t3::Dtype); else y is in the operands' dtype
    uint32_t rows, in, cols, ldw, mt;
    uint32_t wcol0;       // w's first column inside its [in][ldw] array (a member of a joined weight): the array's end,
                          // past which loads bring zeros, lies in * ldw - wcol0 elements from w
    uint32_t ntf, nth;    // column blocks of 256, then of 128
    float* planes;        // PLANES: f32 [K parts][rows][cols], part blockIdx.z's sums
    uint32_t part_steps;  // PLANES: K = 32 steps a part
};

// what a launch ends with: the product in the operands' dtype; format.finishOutput on z = f16(product); or the f32 sums of
// one K part (a launch of few tiles shares K out over grid z so that the GPU fills; the planes are summed in part order
// by the finish launch behind it)
enum GemmEnd : int { kGemmPlain = 0, kGemmFinish = 1, kGemmPlanes = 2 };

template <bool BF16>
__device__ __forceinline__ float4v gemm_mfma(uint4v a, uint4v b, float4v c) {
    if constexpr (BF16)
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
    else
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), c, 0, 0, 0);
}

// Grid (8 mt, ceil(ntf / 8) + ceil(nth / 8)), 512 threads: ntf column blocks of 256 first, then nth of 128 (launched
// last, so they fill the launch's tail: a workgroup holds a compute unit alone, and a last round of full tiles on half
// the compute units would take as long as a full one).
template <bool BF16, int END>
__global__ void __launch_bounds__(512) gemm_half(const GemmArgs a) {
    constexpr bool FINISH = END == kGemmFinish;
    __shared__ __attribute__((aligned(16))) unsigned char smem[kGLds];
    const uint32_t die = blockIdx.x & 7u, mi = blockIdx.x >> 3;
    const uint32_t yf = (a.ntf + 7u) >> 3;
    const bool half = blockIdx.y >= yf;   // uniform over the workgroup
    const uint32_t ni = (half ? blockIdx.y - yf : blockIdx.y) * 8u + die;
    if (ni >= (half ? a.nth : a.ntf)) return;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63u;
    const uint32_t wm = wave & 1u, wn = wave >> 1;
    const uint32_t row0 = mi * kGM, col0 = half ? a.ntf * kGN + ni * (kGN / 2u) : ni * kGN;

    // the tile's windows of x and w: rows past the last one, and the bytes past w's end, read as zeros
    const uint32_t rows_here = a.rows - row0 < kGM ? a.rows - row0 : kGM;
    const uint4v xdesc = rsrc_words(static_cast<const unsigned char*>(a.x) + static_cast<size_t>(row0) * a.in * 2u,
                                   static_cast<uint64_t>(rows_here) * a.in * 2u);
    const uint4v wdesc = rsrc_words(static_cast<const unsigned char*>(a.w) + static_cast<size_t>(col0) * 2u,
                                   (static_cast<uint64_t>(a.in) * a.ldw - a.wcol0 - col0) * 2u);
    // this wave's loads a step: x rows 32 wave .. + 31 (two loads of 16 rows), w rows k = 4 wave .. + 3 (two of 2 rows;
    // a 128-column tile loads 256 columns all the same and leaves the second half alone)
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
    // the K steps this workgroup walks: all of them, or K part blockIdx.z's
    const uint32_t steps_all = a.in / kGK;
    const uint32_t step0 = END == kGemmPlanes ? blockIdx.z * a.part_steps : 0u;
    const uint32_t steps = END == kGemmPlanes ? (steps_all - step0 < a.part_steps ? steps_all - step0 : a.part_steps) : steps_all;
    auto issue = [&](uint32_t step, uint32_t slot) {
        const uint32_t base = lds0 + slot * kGStep, at = step0 + step;
#pragma unroll
        for (uint32_t i = 0; i < 2u; ++i) load_to_lds(xdesc, base + (2u * wave + i) * 1024u, x_voff[i], at * (kGK * 2u));
#pragma unroll
        for (uint32_t i = 0; i < 2u; ++i)
            load_to_lds(wdesc, base + kGXBytes + (2u * wave + i) * 1024u, w_voff[i], at * w_step_bytes);
    };

    // where a lane's fragments sit inside a step's 32 KB
    // activations, row block rb: row 128 wm + 16 rb + lane % 16, piece lane / 16, swizzled
    const uint32_t xf_at = (128u * wm + (lane & 15u)) * 64u + (((lane >> 4) ^ ((lane >> 1) & 3u)) * 16u);
    const uint32_t g = lane >> 4, j = lane & 15u;

    // The K loop and the end for a wave that owns CBN column blocks: 4 (a 256-column tile) or 2 (a 128-column one).
    auto run = [&]<int CBN>() {
        constexpr uint32_t kCols = 64u * CBN;   // the tile's columns
        // weights, column block cb, half h: row k = 8 g + 4 h + j / 4, columns 16 (CBN wn + cb) + 4 (j % 4) .. + 3
        const uint32_t fk = 2u * ((j >> 2) + 4u * (g & 1u));
        uint32_t wf_at[CBN];
#pragma unroll
        for (uint32_t cb = 0; cb < static_cast<uint32_t>(CBN); ++cb) {
            const uint32_t piece = (2u * CBN * wn + 2u * cb + ((j >> 1) & 1u)) ^ fk;
            wf_at[cb] = kGXBytes + (8u * g + (j >> 2)) * 512u + piece * 16u + (j & 1u) * 8u;
        }
        float4v acc[CBN][8];
#pragma unroll
        for (int cb = 0; cb < CBN; ++cb)
#pragma unroll
            for (int rb = 0; rb < 8; ++rb) acc[cb][rb] = float4v{0.f, 0.f, 0.f, 0.f};

#pragma unroll
        for (uint32_t t = 0; t + 1u < kGD; ++t) issue(t, t);   // loads past the last step bring zeros or unused bytes
        wait_loads<static_cast<int>(kGD - 2u) * kGLoadsAStep>();
        __syncthreads();
        uint32_t slot = 0;
        for (uint32_t s = 0; s < steps; ++s) {
            // the slot step s - 1 used is free: every wave passed the barrier that ended it
            issue(s + kGD - 1u, slot == 0u ? kGD - 1u : slot - 1u);
            const unsigned char* st = smem + slot * kGStep;
            uint4v wf[CBN], xf[8];
#pragma unroll
            for (uint32_t cb = 0; cb < static_cast<uint32_t>(CBN); ++cb) {
                const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4v*)(st + wf_at[cb]));
                const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_short4v*)(st + wf_at[cb] + 4u * 512u));
                const uint2 l2 = __builtin_bit_cast(uint2, lo), h2 = __builtin_bit_cast(uint2, hi);
                wf[cb] = uint4v{l2.x, l2.y, h2.x, h2.y};
            }
#pragma unroll
            for (uint32_t rb = 0; rb < 8u; ++rb) xf[rb] = *reinterpret_cast<const uint4v*>(st + xf_at + rb * 1024u);
#pragma unroll
            for (int cb = 0; cb < CBN; ++cb)
#pragma unroll
                for (int rb = 0; rb < 8; ++rb) acc[cb][rb] = gemm_mfma<BF16>(wf[cb], xf[rb], acc[cb][rb]);
            // step s + 1's loads of this wave have landed once at most kGD - 2 steps' are in flight; the barrier then
            // publishes every wave's part of it
            wait_loads<static_cast<int>(kGD - 2u) * kGLoadsAStep>();
            __syncthreads();
            slot = slot + 1u == kGD ? 0u : slot + 1u;
        }
        wait_loads<0>();
        if constexpr (END == kGemmPlanes) {
            // the part's f32 sums as they lie in the accumulators: four adjacent columns of one row a lane and block
            float* plane = a.planes + static_cast<size_t>(blockIdx.z) * a.rows * a.cols;
#pragma unroll
            for (int rb = 0; rb < 8; ++rb)
#pragma unroll
                for (int cb = 0; cb < CBN; ++cb) {
                    const uint32_t row = row0 + 128u * wm + static_cast<uint32_t>(rb) * 16u + (lane & 15u);
                    const uint32_t col = col0 + 16u * CBN * wn + static_cast<uint32_t>(cb) * 16u + 4u * (lane >> 4);
                    if (row < a.rows && col < a.cols)
                        *reinterpret_cast<float4v*>(plane + static_cast<size_t>(row) * a.cols + col) = acc[cb][rb];
                }
            return;
        }
        // every wave is past its last fragment reads (the loop's last barrier) and no load is in flight: the ring's
        // memory takes the output tile. lane: row 16 rb + lane % 16, columns 16 cb + 4 (lane / 16) .. + 3 of the wave's part
        __syncthreads();
#pragma unroll
        for (int rb = 0; rb < 8; ++rb)
#pragma unroll
            for (int cb = 0; cb < CBN; ++cb) {
                const uint32_t row = 128u * wm + static_cast<uint32_t>(rb) * 16u + (lane & 15u);
                const uint32_t col = 16u * CBN * wn + static_cast<uint32_t>(cb) * 16u + 4u * (lane >> 4);
                uint32_t h[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) h[c] = (BF16 && !FINISH) ? bf16_bits(acc[cb][rb][c]) : half_bits(acc[cb][rb][c]);
                *reinterpret_cast<uint2*>(smem + row * kGZRow + col * 2u) = uint2{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
            }
        __syncthreads();
        if constexpr (FINISH) {
            // units = 256 rows x the tile's 128-blocks; a wave takes four a pass
            constexpr uint32_t kBlocks = kCols / 128u, kPasses = 256u * kBlocks / 32u;
            // (unit u = 32 it + 4 wave + lane / 16 is row u / kBlocks, block u % kBlocks: a lane keeps its block, so its
            // eight svh values are loaded once and no pass waits on memory: LDS read, butterflies, store)
            const Row16 g16 = row16(lane);
            const uint32_t q = lane & 15u, blk = (lane >> 4) % kBlocks;
            const uint32_t col = col0 + 128u * blk + 8u * q;
            const bool col_live = col < a.cols;
            float sv[8];
            load8_half(a.svh, col_live ? col : 0u, sv);
#pragma unroll 4
            for (uint32_t it = 0; it < kPasses; ++it) {
                const uint32_t row = (it * 32u + wave * 4u + (lane >> 4)) / kBlocks;
                float v[8];
                load8_half(reinterpret_cast<const uint16_t*>(smem + row * kGZRow), 128u * blk + 8u * q, v);
                finish_row16(v, sv, g16);
                if (col_live && row0 + row < a.rows) store8_act_rt(a.dt, a.y, static_cast<size_t>(row0 + row) * a.cols + col, v);
            }
        } else {
            // 16-byte pieces: a wave stores whole row segments an instruction
            constexpr uint32_t kPieces = kCols / 8u, kPasses = 256u * kPieces / 512u;
            const bool vec = (a.cols & 7u) == 0u;
            for (uint32_t it = 0; it < kPasses; ++it) {
                const uint32_t p = it * 512u + threadIdx.x, row = p / kPieces, piece = p % kPieces;
                const uint32_t col = col0 + piece * 8u;
                if (row0 + row >= a.rows || col >= a.cols) continue;
                const uint4v w = *reinterpret_cast<const uint4v*>(smem + row * kGZRow + piece * 16u);
                uint16_t* dst = static_cast<uint16_t*>(a.y) + static_cast<size_t>(row0 + row) * a.cols + col;
                if (vec) {
                    *reinterpret_cast<uint4v*>(dst) = w;
                } else {
#pragma unroll
                    for (uint32_t c = 0; c < 8u; ++c)
                        if (col + c < a.cols) dst[c] = static_cast<uint16_t>(w[c >> 1] >> (16u * (c & 1u)));
                }
            }
        }
    };
    if (half) run.template operator()<2>();
    else run.template operator()<4>();
}

}  // namespace

namespace {
// The launch's column blocks. Every block 256 wide, except that a launch whose last round of workgroups (one a compute
// unit) would fill at most half the GPU cuts that round's column blocks in two: twice the workgroups, half as long.
GemmArgs gemm_args(const void* x, const void* w, void* y, uint32_t rows, uint32_t in, uint32_t cols, uint32_t ldw,
                   uint32_t wcol0) {
    GemmArgs a{};
    a.x = x;
    a.w = static_cast<const unsigned char*>(w) + static_cast<size_t>(wcol0) * 2u;
    a.wcol0 = wcol0;
    a.y = y;
    a.rows = rows;
    a.in = in;
    a.cols = cols;
    a.ldw = ldw;
    a.mt = (rows + kGM - 1u) / kGM;
    const uint32_t nt = (cols + kGN - 1u) / kGN, cus = 256u;
    const uint32_t last = (a.mt * nt) % cus;          // workgroups of the last round
    uint32_t cut = last != 0u && last <= cus / 2u ? last / a.mt : 0u;   // whole column blocks among them
    if (a.mt * nt < cus) cut = 0u;                    // a launch that never fills the GPU has no tail to balance
    if (cut > nt) cut = nt;
    a.ntf = nt - cut;
    a.nth = 0u;
    if (cut != 0u) {
        const uint32_t first = a.ntf * kGN;           // the cut blocks' first column
        a.nth = (cols - first + kGN / 2u - 1u) / (kGN / 2u);
    }
    return a;
}
dim3 gemm_grid(const GemmArgs& a) { return dim3(8u * a.mt, (a.ntf + 7u) / 8u + (a.nth + 7u) / 8u); }
}  // namespace

// y [rows][cols] = x [rows][in] w[:, wcol0 : wcol0 + cols] for w [in][ldw] (all f16 or all bf16; y row-contiguous). The
// host has checked: in a multiple of 32, ldw and wcol0 multiples of 8, wcol0 + cols within ldw, w and x 16-byte aligned,
// in ldw 2 bytes under 4 GiB. A tile loads 256 columns whatever `cols`: what lies past w's last element reads as zeros.
hipError_t launch_gemm_half(const void* x, const void* w, void* y, uint32_t rows, uint32_t in, uint32_t cols, uint32_t ldw,
                            uint32_t wcol0, bool bf16, hipStream_t s) {
    const GemmArgs a = gemm_args(x, w, y, rows, in, cols, ldw, wcol0);
    const dim3 grid = gemm_grid(a), block(512);
    if (bf16) hipLaunchKernelGGL((gemm_half<true, kGemmPlain>), grid, block, 0, s, a);
    else hipLaunchKernelGGL((gemm_half<false, kGemmPlain>), grid, block, 0, s, a);
    return hipGetLastError();
}

// y [rows][out] = finish(f16(xp [rows][in] w_hat [in][out])) in `dtype`: the W_hat form's product and finish in one
// launch (xp: the prepared rows, f16 in natural order; out a multiple of 128)
hipError_t launch_gemm_finish(const uint16_t* xp, const uint16_t* w_hat, const uint16_t* svh, void* y, uint32_t rows,
                              uint32_t in, uint32_t out, int dtype, hipStream_t s) {
    GemmArgs a = gemm_args(xp, w_hat, y, rows, in, out, out, 0u);
    a.svh = svh;
    a.dt = dtype;
    const dim3 grid = gemm_grid(a), block(512);
    hipLaunchKernelGGL((gemm_half<false, kGemmFinish>), grid, block, 0, s, a);
    return hipGetLastError();
}

// planes f32 [kparts][rows][cols]: part p = the sums over K steps [p part_steps, (p + 1) part_steps) of x w[:, 0:cols]
// (cols a multiple of 4, planes 16-byte aligned); kparts from gemm_kparts
hipError_t launch_gemm_planes(const void* x, const void* w, float* planes, uint32_t rows, uint32_t in, uint32_t cols,
                              uint32_t ldw, uint32_t wcol0, bool bf16, uint32_t kparts, hipStream_t s) {
    GemmArgs a = gemm_args(x, w, nullptr, rows, in, cols, ldw, wcol0);
    if (a.nth != 0u || kparts == 0u || (in / kGK) % kparts != 0u || cols % 4u != 0u) return hipErrorInvalidValue;
    a.planes = planes;
    a.part_steps = (in / kGK) / kparts;
    dim3 grid = gemm_grid(a);
    grid.z = kparts;
    if (bf16) hipLaunchKernelGGL((gemm_half<true, kGemmPlanes>), grid, dim3(512), 0, s, a);
    else hipLaunchKernelGGL((gemm_half<false, kGemmPlanes>), grid, dim3(512), 0, s, a);
    return hipGetLastError();
}

namespace {
// y [rows][cols] in f16 or bf16 = the planes summed in part order, one rounding: the plain product's end over K parts.
// Four adjacent outputs a thread.
template <bool BF16>
__global__ void __launch_bounds__(256) gemm_planes_round(const float* planes, uint16_t* y, uint64_t count4, uint64_t plane,
                                                         uint32_t kparts) {
    const uint64_t i = static_cast<uint64_t>(blockIdx.x) * 256u + threadIdx.x;
    if (i >= count4) return;
    float4v v = *reinterpret_cast<const float4v*>(planes + 4u * i);
    for (uint32_t k = 1; k < kparts; ++k) v += *reinterpret_cast<const float4v*>(planes + k * plane + 4u * i);
    uint32_t h[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) h[c] = BF16 ? bf16_bits(v[c]) : half_bits(v[c]);
    *reinterpret_cast<uint2*>(y + 4u * i) = uint2{h[0] | (h[1] << 16), h[2] | (h[3] << 16)};
}
}  // namespace

hipError_t launch_gemm_planes_round(const float* planes, void* y, uint32_t rows, uint32_t cols, uint32_t kparts, bool bf16,
                                    hipStream_t s) {
    const uint64_t plane = static_cast<uint64_t>(rows) * cols, count4 = plane / 4u;
    const dim3 grid(static_cast<uint32_t>((count4 + 255u) / 256u)), block(256);
    if (bf16) hipLaunchKernelGGL(gemm_planes_round<true>, grid, block, 0, s, planes, static_cast<uint16_t*>(y), count4, plane, kparts);
    else hipLaunchKernelGGL(gemm_planes_round<false>, grid, block, 0, s, planes, static_cast<uint16_t*>(y), count4, plane, kparts);
    return hipGetLastError();
}

}  // namespace t3
