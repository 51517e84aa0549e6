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
// Three launch forms run the same statements in the same order, so their bytes agree (the reference holds its
// one-launch DEC-ONE to its chain the same way, src/core/gpu_test.zig:1016):
//   chain   three launches: dense_prep, dense_gemv<kChain>, dense_finish;
//   arrive  two launches: dense_prep, dense_gemv<kArrive>: the workgroup that completes a 128-column block's planes
//           (an integer arrival counter over device-coherent stores, nothing spins) runs the block's finish;
//   one     one launch, the fewest rows (up to 4 at eight tiles a step, up to 2 at four): dense_gemv<kOne> prepares
//           its own K part in LDS, then as arrive.
// The role of each launch follows the reference's HIP plan (src/hip/plan.zig:161-204); the launch shapes, the lane
// plan and the use of MFMA are this library's own.

#include <type_traits>

#include "t3_gemv_core.hpp"
#include "t3_kernels.hpp"
#include "t3_stages.hpp"

namespace t3 {
namespace {

enum Fuse : int { kChain = 0, kArrive = 1, kOne = 2 };

// Grid (in / 128, rows), 64 threads. xq: [steps][rows][64 bytes], a step R = 1 or 2 input tiles (the GEMV's codebook form
// decides, gemv_step_rows): R 1: word quad_slot(r) of (tile, row) = the f16 value of input 16 tile + r in both halves; R 2:
// the 32 inputs of the tile pair as plain f16 in pair-quad order. The rows of one step lie side by side, so the GEMV's
// fragment of a step (64 bytes a row) is one contiguous piece of whole cache lines (with a row's tiles adjacent instead, a
// 16-row fragment touched 16 lines for half of each, and 32 rows cost the K5 GEMV a third of its time).
// xs: f32 [rows][in / 128].
template <int R>
__global__ void __launch_bounds__(64) dense_prep(const void* x, const uint16_t* suh, uint32_t* xq, float* xs,
                                                 uint32_t in, int dt) {
    const uint32_t b = blockIdx.x, row = blockIdx.y, lane = threadIdx.x;
    uint32_t hv[2];
    float sum;
    prep_values(dt, x, suh, in, row, b, lane, hv, sum);
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
        const uint32_t i = b * 128u + lane + 64u * j, step = i / (16u * R), e = i % (16u * R);
        x_step_store<R>(reinterpret_cast<unsigned char*>(xq) + (static_cast<size_t>(step) * gridDim.y + row) * 64u, e, hv[j]);
    }
    if (lane == 0u) xs[static_cast<size_t>(row) * (in / 128u) + b] = sum;
}

// One wave finishes outputs b 128 + L and + 64 of one row. xs_row: the row's in / 128 block sums. ZCOH / XCOH: the
// planes / the block sums were written by other workgroups of this launch. Loads go out eight at a time and are added
// in slice (or block) order: the sums do not depend on the batching.
template <bool ZCOH, bool XCOH>
__device__ __forceinline__ void finish_block(int dt, const float* z, const float* xs_row, const uint16_t* svh, void* y,
                                             uint32_t out, uint32_t rows, uint32_t ks, uint32_t inblk, int defer,
                                             uint32_t row, uint32_t b, uint32_t lane) {
    auto get_z = [](const float* p) { return ZCOH ? load_coherent(p) : *p; };
    auto get_x = [](const float* p) { return XCOH ? load_coherent(p) : *p; };
    // The deferred map's sum of the row's block sums, 0 + s[0] + s[1] + ... in block order. Up to 64 blocks: one load
    // across the wave's lanes, in flight beside the planes' loads, added up lane by lane afterwards; more: eight at a time.
    float xsum = 0.0f, xmine = 0.0f;
    const bool xwave = defer && inblk <= 64u;
    if (xwave && lane < inblk) xmine = get_x(xs_row + lane);
    if (defer && !xwave)
        for (uint32_t q0 = 0; q0 < inblk; q0 += 8u) {
            float part[8];
#pragma unroll
            for (uint32_t q = 0; q < 8u; ++q) part[q] = q0 + q < inblk ? get_x(xs_row + q0 + q) : 0.0f;
#pragma unroll
            for (uint32_t q = 0; q < 8u; ++q)
                if (q0 + q < inblk) xsum += part[q];
        }
    float v[2];
    const size_t plane = static_cast<size_t>(rows) * out;
    const float* z0 = z + static_cast<size_t>(row) * out + b * 128u + lane;
    float acc[2] = {0.0f, 0.0f};
    for (uint32_t k0 = 0; k0 < ks; k0 += 8u) {
        float part[8][2];
#pragma unroll
        for (uint32_t k = 0; k < 8u; ++k)
#pragma unroll
            for (uint32_t j = 0; j < 2u; ++j) part[k][j] = k0 + k < ks ? get_z(z0 + (k0 + k) * plane + 64u * j) : 0.0f;
#pragma unroll
        for (uint32_t k = 0; k < 8u; ++k)
            if (k0 + k < ks) {
                // the first plane starts the sum (0 + z would turn a -0 into +0)
                acc[0] = k0 + k == 0u ? part[k][0] : acc[0] + part[k][0];
                acc[1] = k0 + k == 0u ? part[k][1] : acc[1] + part[k][1];
            }
    }
    if (xwave)
        for (uint32_t q = 0; q < inblk; ++q)
            xsum += __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, xmine), static_cast<int>(q)));
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
        float s = acc[j];
        if (defer) s = __builtin_fmaf(s, mul1_a(), mul1_b() * xsum);
        v[j] = round_half(s);
    }
    h128_wave(v, lane);
#pragma unroll
    for (uint32_t j = 0; j < 2u; ++j) {
        const uint32_t o = b * 128u + lane + 64u * j;
        store_act_rt(dt, y, static_cast<size_t>(row) * out + o, round_half(v[j] * kHadScale * half_value(svh[o])));
    }
}

// Grid (out / 128, rows), 64 threads.
__global__ void __launch_bounds__(64) dense_finish(const float* z, const float* xs, const uint16_t* svh, void* y,
                                                   uint32_t out, uint32_t rows, uint32_t ks, uint32_t inblk, int defer,
                                                   int dt) {
    finish_block<false, false>(dt, z, xs + static_cast<size_t>(blockIdx.y) * inblk, svh, y, out, rows, ks, inblk, defer,
                        blockIdx.y, blockIdx.x, threadIdx.x);
}

struct GemvArgs {
    const uint32_t* w;
    const uint32_t* xq;   // kChain, kArrive: the prepared rows
    float* z;
    float* xs;            // block sums: [rows][in / 128]; kOne: [out / 128][rows][in / 128], a copy a column block,
                          // each written by that block's own workgroups (one shared copy would be stored to by
                          // every workgroup at once: 3,000 coherent stores to one cache line serialise for ~80 us)
    const void* x;        // kOne: the raw activations
    const uint16_t* suh;  // kOne
    const uint16_t* svh;  // kArrive, kOne
    void* y;              // kArrive, kOne
    uint32_t* arrive;     // kArrive, kOne: one counter a 128-column block, zero between calls
    uint32_t in, out, rows, n, wbits, per, ks;
    int dt, defer;
};

// Grid (out / 16 / BT, KS), 256 threads (4 waves). A workgroup owns BT adjacent output tiles and K slice blockIdx.y;
// wave sg takes part sg of the slice, `per` = in_tiles / (4 KS) input tiles (the host divides: the GPU has no scalar
// divide). RB = 16-row blocks of x (1 or 2). z f32 [KS][rows][out]: the four waves' sums, wave 0 first.
// LDS: the tiles go from memory straight into an LDS ring (served where a wave's walk is long, dense_gemv_lds_ring);
// else through the register ring.
// A persistent form of this grid (a workgroup looping over two or three column blocks, everything else unchanged) was
// measured at 4096 x 12288 K4, one row: 14.9 us a call with 768 workgroups of one block each, 20.3 with 384 of two, 25.4
// with 256 of three. Every workgroup of the launch is resident from its first cycle as it is; fewer, longer ones only
// put the column blocks' chains of round trips (first bytes, hand-off, finish) one behind the other.
template <int CB, int WIDE, int RB, int BT, int FUSE, bool LDS>
__global__ void __launch_bounds__(256) dense_gemv(const GemvArgs a) {
    typedef GemvStream<LDS, CB, WIDE, RB, BT, XLds> StreamL;
    typedef GemvStream<LDS, CB, WIDE, RB, BT, XGlobal> StreamG;
    constexpr uint32_t kStage = StreamG::kStageBytes;
    constexpr int R = gemv_step_rows<CB>();   // tile rows a step
    // MUL1's map is deferred exactly under that codebook form (a.defer repeats it): the other forms' kernels carry none
    // of its block sums
    constexpr bool kDefer = CB == kMul1Defer;
    constexpr uint32_t kRed = 4u * RB * BT * 64u * 16u;
    constexpr uint32_t kMain = kRed > 4u * kStage ? kRed : 4u * kStage;
    // the waves' LDS rings while they stream; the four waves' partial sums afterwards
    __shared__ __attribute__((aligned(16))) unsigned char smem[kMain];
    __shared__ uint32_t last_flag;
    float4v(*red)[RB * BT * 64] = reinterpret_cast<float4v(*)[RB * BT * 64]>(smem);
    const uint32_t blk = blockIdx.x, ksl = blockIdx.y;
    const uint32_t sg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63u;
    const uint32_t out_tiles = a.out >> 4, nw = a.n >> 1, rows = a.rows, per = a.per;
    const uint32_t tk0 = (ksl * 4u + sg) * per;

    float4v acc[RB][BT];
#pragma unroll
    for (int r = 0; r < RB; ++r)
#pragma unroll
        for (int t = 0; t < BT; ++t) acc[r][t] = float4v{0.f, 0.f, 0.f, 0.f};

    const uint64_t wstride = static_cast<uint64_t>(out_tiles) * nw;  // words a tile row
    const uint32_t* wbase = a.w + static_cast<uint64_t>(blk) * BT * nw + tk0 * wstride;
    const uint32_t wstep = static_cast<uint32_t>(wstride) * 4u;

    // x fragment: activation row (lane % 16) of block r, K slots 8g..8g+7 = quad g's four inputs, each doubled.
    // Rows past the call's last are zeros (the chain forms) or alias row 0 (the one-launch form): their sums are
    // computed and never stored.
    uint32_t xoff[RB];
    constexpr uint32_t kShare = 8u / BT;  // workgroup columns a 128-column block
    const uint32_t b128 = blk / kShare;
    const uint32_t inblk = a.in / 128u;
    if constexpr (FUSE == kOne) {
        static_assert(FUSE != kOne || RB == 1, "the one-launch form serves up to 4 rows");
        extern __shared__ __attribute__((aligned(16))) unsigned char xdyn[];
        const uint32_t steps = per / R;
        unsigned char* xst = xdyn + sg * ((steps + 1u) * (kXldsRows * 64u));
        const uint32_t row = lane & 15u;
        xoff[0] = (row < rows ? row : 0u) * 64u + (lane >> 4) * 16u;
        StreamL stream(wbase, wstep, per, a.n, a.wbits, XLds{xst}, xoff, smem + sg * kStage, lane);
        // The register ring's loads are the compiler's own, and a wave's loads come back in the order they went out: the
        // activations' go out first, so the prepare waits for nothing but them (behind the codes' first tile rows it
        // began later: the call 14.8 -> 14.6 us at one row, 16.2 -> 15.7 at four). The LDS ring's loads are issued from
        // asm and not counted by the compiler, which then waits for every load in flight whichever went first.
        constexpr bool kXFirst = !LDS;
        if constexpr (!kXFirst) stream.issue();
        // While the codes fly, the wave prepares its own K part: per / 8 whole 128-blocks a row, the statements of
        // dense_prep, into its LDS x stage [steps + 1][4][64 bytes] (the last step zeros). The block sums go to the
        // column block's own copy of xs (deferred MUL1 map only; the block's second workgroup column, if any, would
        // store the same values again).
        // Every row's loads go out together (rows past the call's alias the last real one, so there is no branch among
        // the loads): a further row then costs its butterfly, not another round trip. One row and one block a wave, the
        // commonest call, has a copy of its own that loads nothing else (a load costs the wave its issue whether its
        // value is used or not: 20 loads in front of the codes' held them back 0.6 us where 4 do the work).
        const uint32_t blocks = per >> 3;  // 1 or 2
        auto prepare = [&](auto nr_c, auto nb_c) {
            constexpr uint32_t NR = decltype(nr_c)::value, NB = decltype(nb_c)::value;  // rows loaded, blocks a wave
            float raw[NR][NB][2], sc[NB][2];
            auto load_rows = [&](auto tag) {
                constexpr int DT = decltype(tag)::value;
#pragma unroll
                for (uint32_t b = 0; b < NB; ++b)
#pragma unroll
                    for (uint32_t j = 0; j < 2u; ++j) {
                        const uint32_t i = ((tk0 >> 3) + b) * 128u + lane + 64u * j;
                        sc[b][j] = half_value(a.suh[i]);
#pragma unroll
                        for (uint32_t r = 0; r < NR; ++r)
                            raw[r][b][j] = load_act<DT>(a.x, static_cast<size_t>(r < rows ? r : rows - 1u) * a.in + i);
                    }
            };
            if (a.dt == kF32) load_rows(std::integral_constant<int, kF32>{});
            else if (a.dt == kF16) load_rows(std::integral_constant<int, kF16>{});
            else load_rows(std::integral_constant<int, kBf16>{});
            if constexpr (kXFirst) {
                __builtin_amdgcn_sched_barrier(0);
                stream.issue();
                __builtin_amdgcn_sched_barrier(0);
            }
#pragma unroll
            for (uint32_t r = 0; r < NR; ++r) {
                if (r >= rows) break;
#pragma unroll
                for (uint32_t b = 0; b < NB; ++b) {
                    float v[2] = {round_half(raw[r][b][0]) * sc[b][0], round_half(raw[r][b][1]) * sc[b][1]};
                    uint32_t hv[2];
                    float sum;
                    prep_core(v, lane, hv, sum, kDefer);
#pragma unroll
                    for (uint32_t j = 0; j < 2u; ++j) {
                        const uint32_t i = b * 128u + lane + 64u * j;  // element of the wave's K part: step i / (16 R)
                        x_step_store<R>(xst + ((i / (16u * R)) * kXldsRows + r) * 64u, i % (16u * R), hv[j]);
                    }
                    if (kDefer && lane == 0u && blk % kShare == 0u)
                        store_coherent(a.xs + (static_cast<size_t>(b128) * rows + r) * inblk + (tk0 >> 3) + b, sum);
                }
            }
        };
        typedef std::integral_constant<uint32_t, 1u> One;
        typedef std::integral_constant<uint32_t, 2u> Two;
        typedef std::integral_constant<uint32_t, kXldsRows> Rows;
        if (rows == 1u) {
            if (blocks == 1u) prepare(One{}, One{});
            else prepare(One{}, Two{});
        } else {
            if (blocks == 1u) prepare(Rows{}, One{});
            else prepare(Rows{}, Two{});
        }
        for (uint32_t i = lane; i < kXldsRows * 16u; i += 64u)
            *reinterpret_cast<uint32_t*>(xst + steps * (kXldsRows * 64u) + i * 4u) = 0u;
        stream.run(acc);
    } else {
#pragma unroll
        for (int r = 0; r < RB; ++r) {
            const uint32_t row = static_cast<uint32_t>(r) * 16u + (lane & 15u);
            xoff[r] = x_frag_offset(lane, row < rows, row * 64u);
        }
        StreamG stream(wbase, wstep, per, a.n, a.wbits,
                       XGlobal{a.xq, static_cast<uint64_t>(rows) * (a.in / (16u * R)) * 64u, (tk0 / R) * rows * 64u, rows * 64u},
                       xoff, smem + sg * kStage, lane);
        stream.issue();
        stream.run(acc);
    }
    __syncthreads();  // every wave is done with its rings (no load in flight) before the sums take the memory

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
        float* dst = a.z + (static_cast<size_t>(ksl) * rows + row) * a.out + (blk * BT + t) * 16u + 4u * (l >> 4);
        if constexpr (FUSE == kChain) {
            *reinterpret_cast<float4v*>(dst) = s;
        } else {
            store_coherent4(dst, s);
        }
    }

    if constexpr (FUSE != kChain) {
        // The last workgroup to arrive at a 128-column block finishes it. The planes (and the one-launch form's block
        // sums) are stored device-coherently; once every lane's stores are acknowledged the workgroup counts itself
        // in, and the one that reads the full count sums the planes in slice order, as dense_finish does. Nothing
        // spins, and no cache is flushed.
        wait_stores();
        __syncthreads();
        if (threadIdx.x == 0u) {
            const uint32_t before =
                __hip_atomic_fetch_add(a.arrive + arrive_slot(b128, a.out / 128u), 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last_flag = before == a.ks * kShare - 1u;
        }
        __syncthreads();
        if (last_flag) {
            for (uint32_t row = sg; row < rows; row += 4u) {
                const float* xs_row = a.xs + (FUSE == kOne ? (static_cast<size_t>(b128) * rows + row) * inblk
                                                           : static_cast<size_t>(row) * inblk);
                // arrive form: the block sums came from the prepare launch, only the planes cross workgroups
                finish_block<true, FUSE == kOne>(a.dt, a.z, xs_row, a.svh, a.y, a.out, rows, a.ks, inblk, kDefer ? 1 : 0, row,
                                                 b128, lane);
            }
            if (threadIdx.x == 0u)  // zero again for the next call
                __hip_atomic_store(a.arrive + arrive_slot(b128, a.out / 128u), 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
    }
}

template <int CB, int WIDE, int RB, int BT>
hipError_t launch_gemv_fuse(const DenseLaunch& d, int fuse, hipStream_t s) {
    GemvArgs a;
    a.w = d.trellis;
    a.xq = d.xq;
    a.z = d.z;
    a.xs = d.xs;
    a.x = d.x;
    a.suh = d.suh;
    a.svh = d.svh;
    a.y = d.y;
    a.arrive = d.arrive;
    a.in = d.in;
    a.out = d.out;
    a.rows = d.rows;
    a.n = d.n;
    a.wbits = d.wbits;
    a.per = (d.in / 16u) / (4u * d.ks);
    a.ks = d.ks;
    a.dt = d.dtype;
    a.defer = d.codebook == kMul1Defer;
    const dim3 grid((d.out / 16u) / BT, d.ks), block(256);
    const bool lds = dense_gemv_lds_ring(a.per);
    if (fuse == kOne) {
        if constexpr (RB == 1) {
            // (the one-launch form serves waves of 8 or 16 tile rows: below the LDS ring's served bound)
            const size_t dyn = 4u * (a.per / gemv_step_rows<CB>() + 1u) * (kXldsRows * 64u);
            if (lds) hipLaunchKernelGGL((dense_gemv<CB, WIDE, 1, BT, kOne, true>), grid, block, dyn, s, a);
            else hipLaunchKernelGGL((dense_gemv<CB, WIDE, 1, BT, kOne, false>), grid, block, dyn, s, a);
        } else {
            return hipErrorInvalidValue;
        }
    } else if (fuse == kArrive) {
        if (lds) hipLaunchKernelGGL((dense_gemv<CB, WIDE, RB, BT, kArrive, true>), grid, block, 0, s, a);
        else hipLaunchKernelGGL((dense_gemv<CB, WIDE, RB, BT, kArrive, false>), grid, block, 0, s, a);
    } else {
        if (lds) hipLaunchKernelGGL((dense_gemv<CB, WIDE, RB, BT, kChain, true>), grid, block, 0, s, a);
        else hipLaunchKernelGGL((dense_gemv<CB, WIDE, RB, BT, kChain, false>), grid, block, 0, s, a);
    }
    return hipGetLastError();
}

// ---- the LDS-table decoder, measured (build with -DT3_GEMV_TABLE_FROM=<tile rows a wave> to route the chain's GEMV of a
// matrix whose waves walk at least that many tile rows here; off in the served build) ---------------------------
// One workgroup of twelve waves a compute unit holds the f16 weight of every 16-bit codeword in LDS (128 KB of the
// 160) and runs three of dense_gemv's four-wave workgroups at a time beside it, persistently: virtual workgroup
// (column block, K slice) v = (pass x grid + workgroup) x 3 + group. T3_GEMV_TABLE_PAIRS of a lane's four weight
// registers a tile pair are looked up (two vector operations and a ds_read_u16 a weight), the others hashed (four
// vector operations): the two pipes side by side. The K partition, the order of the waves' sums and so the planes' bytes
// are dense_gemv's. Up to four rows, up to four bits a weight (a tile of whole 16-byte pieces within 128 bytes), MCG.
#ifndef T3_GEMV_TABLE_FROM
#define T3_GEMV_TABLE_FROM 0xFFFFFFFFu
#endif
constexpr uint32_t kTabTableBytes = 131072u, kTabWaves = 12u, kTabRows = 4u;

template <int BT>
__global__ void __launch_bounds__(768) dense_gemv_tab(const GemvArgs a, uint32_t nblk, uint32_t nvwg, uint32_t iters) {
    typedef GemvStreamTab<BT, 2> Stream;
    constexpr uint32_t kStage = Stream::kStageBytes;
    static_assert(4u * kStage >= 4u * kTabRows * BT * 4u * 16u, "a group's sums fit its four stages");
    unsigned char* stages = t3_table_lds + kTabTableBytes;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), g = wave >> 2, sg = wave & 3u;
    const uint32_t lane = threadIdx.x & 63u, gtid = threadIdx.x & 255u;
    uint32_t* tab32 = reinterpret_cast<uint32_t*>(t3_table_lds);
    for (uint32_t i = threadIdx.x; i < 32768u; i += 768u)
        tab32[i] = static_cast<uint32_t>(decode_mcg(2u * i)) | (static_cast<uint32_t>(decode_mcg(2u * i + 1u)) << 16);
    __syncthreads();
    const uint32_t out_tiles = a.out >> 4, nw = a.n >> 1, rows = a.rows, per = a.per;
    const uint64_t wstride = static_cast<uint64_t>(out_tiles) * nw;
    const uint32_t wstep = static_cast<uint32_t>(wstride) * 4u;
    float4v* red = reinterpret_cast<float4v*>(stages + g * 4u * kStage);  // [wave][row][tile][lane / 16]
    for (uint32_t it = 0; it < iters; ++it) {
        const uint32_t v = (it * gridDim.x + blockIdx.x) * 3u + g;
        const bool live = v < nvwg;  // uniform over the group's waves
        const uint32_t vv = live ? v : 0u, ksl = vv / nblk, blk = vv - ksl * nblk;
        float4v acc[1][BT];
#pragma unroll
        for (int t = 0; t < BT; ++t) acc[0][t] = float4v{0.f, 0.f, 0.f, 0.f};
        if (live) {
            const uint32_t tk0 = (ksl * 4u + sg) * per;
            const uint32_t* wbase = a.w + static_cast<uint64_t>(blk) * BT * nw + tk0 * wstride;
            const uint32_t xoff = x_frag_offset(lane, (lane & 15u) < rows, (lane & 15u) * 64u);
            Stream stream(wbase, wstep, per, a.n, a.wbits,
                          XGlobal{a.xq, static_cast<uint64_t>(rows) * (a.in / 32u) * 64u, (tk0 / 2u) * rows * 64u, rows * 64u},
                          xoff, stages + wave * kStage, lane);
            stream.issue();
            stream.run(acc);
        }
        __syncthreads();  // every wave is done with its stage before the sums take the memory
        if ((lane & 15u) < rows)
#pragma unroll
            for (int t = 0; t < BT; ++t)
                red[((sg * kTabRows + (lane & 15u)) * BT + static_cast<uint32_t>(t)) * 4u + (lane >> 4)] = acc[0][t];
        __syncthreads();
        if (live && gtid < rows * BT * 4u) {
            const uint32_t row = gtid / (BT * 4u), t = (gtid >> 2) % BT, q = gtid & 3u;
            const uint32_t at = (row * BT + t) * 4u + q, wv = kTabRows * BT * 4u;
            const float4v s = ((red[at] + red[wv + at]) + red[2u * wv + at]) + red[3u * wv + at];
            *reinterpret_cast<float4v*>(a.z + (static_cast<size_t>(ksl) * rows + row) * a.out + (blk * BT + t) * 16u + 4u * q) = s;
        }
        __syncthreads();  // the sums are read before the next pass stages its first tile rows
    }
}

inline bool gemv_table_serves(const DenseLaunch& d, int fuse) {
    const uint32_t per = (d.in / 16u) / (4u * d.ks);
    return fuse == kFuseChain && d.codebook == kMcg && per >= T3_GEMV_TABLE_FROM && d.rows <= kTabRows && d.n <= 64u &&
           d.n % 8u == 0u && (d.out / 16u) % 4u == 0u;
}

hipError_t launch_gemv_tab(const DenseLaunch& d, hipStream_t s) {
    constexpr int BT = 4;
    GemvArgs a{};
    a.w = d.trellis;
    a.xq = d.xq;
    a.z = d.z;
    a.in = d.in;
    a.out = d.out;
    a.rows = d.rows;
    a.n = d.n;
    a.wbits = d.wbits;
    a.per = (d.in / 16u) / (4u * d.ks);
    a.ks = d.ks;
    const uint32_t nblk = (d.out / 16u) / BT, nvwg = nblk * d.ks;
    const uint32_t grid = (nvwg + 2u) / 3u < 256u ? (nvwg + 2u) / 3u : 256u;
    const uint32_t iters = (nvwg + grid * 3u - 1u) / (grid * 3u);
    const uint32_t dyn = kTabTableBytes + kTabWaves * GemvStreamTab<BT, 2>::kStageBytes;
    static bool allowed = false;  // once a process: the launch may take more than 64 KB of dynamic LDS
    if (!allowed) {
        if (const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(&dense_gemv_tab<BT>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(dyn));
            e != hipSuccess)
            return e;
        allowed = true;
    }
    hipLaunchKernelGGL((dense_gemv_tab<BT>), dim3(grid), dim3(768), dyn, s, a, nblk, nvwg, iters);
    return hipGetLastError();
}

template <int CB>
hipError_t launch_gemv_cb(const DenseLaunch& d, int fuse, hipStream_t s) {
    const bool two = d.rows > 16u;
    return with_reader(d.n, [&](auto reader) {
        constexpr int R = decltype(reader)::value;
        if constexpr (R == kNarrow) {
            if (d.bt == 8u) return two ? launch_gemv_fuse<CB, R, 2, 8>(d, fuse, s) : launch_gemv_fuse<CB, R, 1, 8>(d, fuse, s);
        }
        // a wide rate's tile is over 128 bytes: eight of them never fit a load, the host gives them four
        if (d.bt != 4u && R != kNarrow) return hipErrorInvalidValue;
        return two ? launch_gemv_fuse<CB, R, 2, 4>(d, fuse, s) : launch_gemv_fuse<CB, R, 1, 4>(d, fuse, s);
    });
}

}  // namespace

namespace {
// y[row][c] = dtype(y[row][c] + bias[c]): grid (ceil(out / 256), rows), 256 threads
__global__ void __launch_bounds__(256) bias_add(void* y, const void* bias, uint32_t out, int dt) {
    const uint32_t c = blockIdx.x * 256u + threadIdx.x;
    if (c >= out) return;
    const size_t at = static_cast<size_t>(blockIdx.y) * out + c;
    store_act_rt(dt, y, at, load_act_rt(dt, y, at) + load_act_rt(dt, bias, c));
}
}  // namespace

hipError_t launch_bias_add(void* y, const void* bias, uint32_t rows, uint32_t out, int dtype, hipStream_t s) {
    for (uint32_t r0 = 0; r0 < rows; r0 += 65535u) {  // grid.y holds 65535 rows a launch
        const uint32_t part = rows - r0 < 65535u ? rows - r0 : 65535u;
        void* yp = static_cast<unsigned char*>(y) + static_cast<size_t>(r0) * out * (dtype == kF32 ? 4u : 2u);
        hipLaunchKernelGGL(bias_add, dim3((out + 255u) / 256u, part), dim3(256), 0, s, yp, bias, out, dtype);
        if (const hipError_t e = hipGetLastError(); e != hipSuccess) return e;
    }
    return hipSuccess;
}

hipError_t launch_dense_prep(const DenseLaunch& d, hipStream_t s) {
    // the layout the GEMV of this codebook form reads
    const bool two = d.codebook == kMcg || d.codebook == kMul1;
    static_assert(gemv_step_rows<kMcg>() == 2 && gemv_step_rows<kMul1>() == 2 && gemv_step_rows<kMcgPair>() == 1 &&
                  gemv_step_rows<kMul1Defer>() == 1);
    if (two) hipLaunchKernelGGL(dense_prep<2>, dim3(d.in / 128u, d.rows), dim3(64), 0, s, d.x, d.suh, d.xq, d.xs, d.in, d.dtype);
    else hipLaunchKernelGGL(dense_prep<1>, dim3(d.in / 128u, d.rows), dim3(64), 0, s, d.x, d.suh, d.xq, d.xs, d.in, d.dtype);
    return hipGetLastError();
}

hipError_t launch_dense_gemv(const DenseLaunch& d, int fuse, hipStream_t s) {
    if (gemv_table_serves(d, fuse)) return launch_gemv_tab(d, s);
    switch (d.codebook) {
        case kMul1: return launch_gemv_cb<kMul1>(d, fuse, s);
        case kMcg: return launch_gemv_cb<kMcg>(d, fuse, s);
        case kMul1Defer: return launch_gemv_cb<kMul1Defer>(d, fuse, s);
        default: return launch_gemv_cb<kMcgPair>(d, fuse, s);
    }
}

hipError_t launch_dense_finish(const DenseLaunch& d, hipStream_t s) {
    hipLaunchKernelGGL(dense_finish, dim3(d.out / 128u, d.rows), dim3(64), 0, s, d.z, d.xs, d.svh, d.y, d.out, d.rows,
                       d.ks, d.in / 128u, static_cast<int>(d.codebook == kMul1Defer), d.dtype);
    return hipGetLastError();
}

}  // namespace t3
