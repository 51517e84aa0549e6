// Above the decode rows on gfx950: the grouped trellis GEMM on the matrix cores, the route that feeds it, and the two
// chains it serves: routed experts beyond 16 rows (turboexl3 src/core/prefill.zig:1-24; roles of src/hip/plan.zig:
// 380-520) and one dense projection beyond 32 rows (src/core/dense.zig:978-1034).
//
// The GEMM. An item is up to RB * 16 activation rows that share one weight matrix (one expert's rows after the route,
// or a block of a dense call's rows). A workgroup takes one item and 256 output columns; each of its four waves owns
// four adjacent 16 x 16 tiles a tile row and decodes them EXACTLY (the f16 bits of format.decodeTile), a quad of
// weights a lane, two tile rows a step: 8 f16 = the A fragment of v_mfma_f32_16x16x32_f16 over K = 32, with no shuffle
// and no LDS round trip for the decoded weights. The item's prepared activations (f16, quad order) go through LDS once
// a step for all four waves and are read back as B fragments, 16 bytes a lane. Every decoded weight feeds RB MFMAs.
// A row's sums depend on (matrix, K order) alone: not on the item it landed in, nor on the rows beside it.
//
// Cost (measured beside the GEMV): the exact decode is ~5 vector-ALU operations a weight and the matrix core does not
// overlap them, so at 64 rows an item the kernel is bound by the decode, not by MFMA.

#include "t3_decode.hpp"
#include "t3_kernels.hpp"
#include "t3_lds_loads.hpp"
#include "t3_routed.hpp"
#include "t3_stages.hpp"

namespace t3 {
namespace {

constexpr uint32_t kPfSlot = 256;   // LDS bytes a tile's words take (a tile is at most 256 bytes)
constexpr uint32_t kPfTiles = 4;    // adjacent tiles a wave
constexpr uint32_t kPfWaveStep = 2u * kPfTiles * kPfSlot;  // LDS bytes of a wave's weight words a step (two tile rows)

struct PfGemm {
    const uint32_t* w[2];    // the bank's trellis a projection (gate, up) or (down, -)
    const uint32_t* ws[2];   // the shared bank's: experts numbered from `experts` up
    const uint16_t* xq[2];   // prepared activations f16 [positions][in], pair-quad order
    float* z[2];             // f32 [positions][out]
    const uint32_t* items;   // {expert, first position, rows, 0} an item; null: dense, item i = rows i RB 16 ...
    const uint32_t* n_items; // the route's item count (device)
    uint32_t in, out, n, wbits, positions, experts, nblk;  // nblk: workgroup columns (256 output columns each)
    uint32_t spread;  // dies one item's column blocks go round: 1 with eight items or more a launch, up to 8 with one
    uint32_t kparts;  // K parts (grid z): part k multiplies its share of the tile rows into plane k of z
    uint32_t plane;   // elements between z's planes
    uint32_t zhalf;   // z holds f16 [positions][out] (the sums rounded at the launch's end) instead of f32: one K part, and
                      // a finish that starts by rounding them (not GLM's profile)
    const float* xtot[2];  // zhalf under MUL1's deferred map: a position's total of its input's block sums (pf_rowsums);
                           // the launch's end applies the map before it rounds. Null: no map.
};

// Grid (8 * ceil(nblk / spread) * ceil(max_items / (8 / spread)), projections, kparts), 256 threads. Consecutive
// workgroup ids go round the eight dies, so the workgroups that share an item's activations (its nblk column blocks)
// are given ids 8 apart: one die's L2 serves them all. With fewer than eight items that would leave dies idle (one item:
// seven of eight), so an item's column blocks then go round `spread` dies.
//
// Shapes: RB 16-row blocks an item, four adjacent tiles a wave, 256 columns a workgroup. RB 4: 64 rows. RB 8: 128 rows:
// a decoded weight feeds twice the MFMAs, and an expert with 65-128 rows stays one item (a second, short item would
// pay the whole decode again). RB 2: 32 rows for sparse routings. Row blocks past the item's last row skip their MFMAs.
//
// The operands reach LDS without passing through registers, D steps deep (a step = K 32 = two tile rows):
//   weights      a wave's four tiles of a tile row, one load: lane L brings bytes 16 (L % 16).. of tile L / 16 to the
//                tile's 256-byte slot; each lane then reads back the two words its quad's windows span (four where a wide
//                rate's quads pass two words);
//   activations  the item's rows, 64 bytes a row a step, 16 rows a load. Row r's 16-byte piece p is kept at position
//                p ^ ((r >> 1) & 3) of the row, which spreads a B fragment's reads (16 rows, one piece each) over the
//                banks at row stride 64 (measured: 4.2 cycles a wave's read, 8 unswizzled).
// Measured before this form, with loads held in registers one step ahead: the kernel waited on the weight loads 12 %
// of its time (strided 256-byte pieces come back slower than one step takes).
//
// LBMAX < RB (the 128-row shape only): the same kernel with accumulators for LBMAX live row blocks (16 LBMAX registers
// a lane instead of 128) and rings three steps deep, which fits three waves a SIMD where the full shape fits two. It
// serves routings whose items the route cuts at 16 LBMAX = 96 rows (src: `moe_item_rows`).
template <int CB, int WIDE, int RB, int LBMAX = RB>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(LBMAX < RB ? 3 : 1, 8))) pf_gemm(const PfGemm a) {
    constexpr bool kShort = LBMAX < RB;
    constexpr uint32_t D = (RB == 2 || kShort) ? 3u : 4u;    // steps in flight + 1
    constexpr uint32_t BM = RB * 16u;
    constexpr uint32_t kAStep = BM * 64u;                     // LDS bytes of the item's rows a step
    constexpr uint32_t kALoads = RB >= 4 ? RB / 4u : 1u;      // activation loads a wave a step (16 rows each)
    constexpr int kPerStep = static_cast<int>(kALoads) + 2;   // loads a wave a step
    __shared__ __attribute__((aligned(16))) unsigned char smem[D * kAStep + 4u * D * kPfWaveStep];
    static_assert(sizeof(smem) <= 65536u, "the LDS addresses of the loads are 16 bits");

    const uint32_t id = blockIdx.x, proj = blockIdx.y, kpart = blockIdx.z;
    const uint32_t die = id & 7u, j = id >> 3, nbs = (a.nblk + a.spread - 1u) / a.spread;
    const uint32_t blk = (j % nbs) * a.spread + die % a.spread, item_i = (j / nbs) * (8u / a.spread) + die / a.spread;
    if (blk >= a.nblk) return;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63u;
    uint32_t e = 0, first, count;
    if (a.items) {
        if (item_i >= a.n_items[0]) return;
        e = a.items[item_i * 4u];
        first = a.items[item_i * 4u + 1u];
        count = a.items[item_i * 4u + 2u];
    } else {
        first = item_i * BM;
        if (first >= a.positions) return;
        count = a.positions - first < BM ? a.positions - first : BM;
    }
    const uint32_t in_tiles = a.in >> 4, out_tiles = a.out >> 4, nw = a.n >> 1;
    const bool from_shared = e >= a.experts;
    const uint32_t* wmat = (from_shared ? a.ws[proj] : a.w[proj]) +
                           static_cast<size_t>(from_shared ? e - a.experts : e) * in_tiles * out_tiles * nw;
    const uint32_t col0 = (blk * 4u + wave) * kPfTiles;  // the wave's first tile column
    const bool active = col0 < out_tiles;               // uniform over the wave (out is a multiple of 128, not of 256)
    const uint32_t wstep = out_tiles * nw * 4u;
    const uint32_t tile_bytes = 2u * a.n, chunk_bytes = kPfTiles * tile_bytes;
    // the wave's window of the matrix: a tile row past the last one falls outside it and reads as zeros
    const uint4v wdesc = rsrc_words(wmat + static_cast<size_t>(col0) * nw,
                                    active ? (in_tiles - 1u) * wstep + chunk_bytes : 0u);
    const uint4v xdesc = rsrc_words(a.xq[proj], static_cast<uint64_t>(a.positions) * a.in * 2u);
    const uint32_t w_voff = (lane & 15u) * 16u < tile_bytes ? (lane >> 4) * tile_bytes + (lane & 15u) * 16u : 0x80000000u;

    const uint32_t lds0 = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(smem));
    const uint32_t a_lds = lds0, w_lds = lds0 + D * kAStep + wave * (D * kPfWaveStep);
    const unsigned char* a_ring = smem;
    const unsigned char* w_ring = smem + D * kAStep + wave * (D * kPfWaveStep);

    // the pieces of the item's rows this lane brings: load i of the wave covers rows 16 (4 i + wave) .. + 15 (RB 2 has
    // two loads' worth of rows: waves 2 and 3 repeat the loads of waves 0 and 1)
    const uint32_t wq = RB == 2 ? (wave & 1u) : wave;
    uint32_t a_voff[kALoads];
#pragma unroll
    for (uint32_t i = 0; i < kALoads; ++i) {
        const uint32_t row = (4u * i + wq) * 16u + (lane >> 2), piece = (lane & 3u) ^ ((row >> 1) & 3u);
        a_voff[i] = row < count ? ((first + row) * a.in + piece * 8u) * 2u : 0x80000000u;
    }
    // this part's steps: the host gives every part an even number of them (in is a multiple of 128)
    const uint32_t steps = (in_tiles >> 1) / a.kparts, step0 = kpart * steps;
    float* z = a.z[proj] + static_cast<size_t>(kpart) * a.plane;
    auto issue = [&](uint32_t step, uint32_t slot) {
#pragma unroll
        for (uint32_t i = 0; i < kALoads; ++i)
            load_to_lds(xdesc, a_lds + slot * kAStep + (4u * i + wq) * 1024u, a_voff[i], (step0 + step) * 64u);
#pragma unroll
        for (uint32_t r = 0; r < 2u; ++r)
            load_to_lds(wdesc, w_lds + slot * kPfWaveStep + r * (kPfTiles * kPfSlot), w_voff,
                        (2u * (step0 + step) + r) * wstep);
    };

    const QuadPlan<WIDE> plan = quad_plan<WIDE>(a.n, lane);
    const uint32_t get_bp = plan.ib_prev * 4u, get_bl = plan.ib_last * 4u;
    const uint32_t get_ap = plan.ia_prev * 4u, get_al = plan.ia_last * 4u;
    auto fetch_w = [&](QuadWords<WIDE>(&wd)[2][kPfTiles], uint32_t slot) {
        const unsigned char* st = w_ring + slot * kPfWaveStep;
#pragma unroll
        for (uint32_t r = 0; r < 2u; ++r)
#pragma unroll
            for (uint32_t t = 0; t < kPfTiles; ++t) {
                const unsigned char* tile = st + (r * kPfTiles + t) * kPfSlot;
                wd[r][t].b_prev = *reinterpret_cast<const uint32_t*>(tile + get_bp);
                wd[r][t].b_last = *reinterpret_cast<const uint32_t*>(tile + get_bl);
                if constexpr (WIDE == kWide) {
                    wd[r][t].a_prev = *reinterpret_cast<const uint32_t*>(tile + get_ap);
                    wd[r][t].a_last = *reinterpret_cast<const uint32_t*>(tile + get_al);
                }
            }
    };
    // the B fragment of block mb: row 16 mb + lane % 16, K slots 8 (lane / 16) ..: its swizzled piece
    const uint32_t b_at = (lane & 15u) * 64u + (((lane >> 4) ^ ((lane >> 1) & 3u)) * 16u);


    // The K loop and the stores for an item of LB live 16-row blocks: no branch inside the loop.
    auto run = [&]<int LB>() {
        float4v acc[LB][kPfTiles];
#pragma unroll
        for (int mb = 0; mb < LB; ++mb)
#pragma unroll
            for (uint32_t t = 0; t < kPfTiles; ++t) acc[mb][t] = float4v{0.f, 0.f, 0.f, 0.f};

        // one step: K = 32 = tile rows 2 step and 2 step + 1
        auto compute = [&](const QuadWords<WIDE>(&wd)[2][kPfTiles], uint32_t slot) {
            uint4v bf[LB];
#pragma unroll
            for (int mb = 0; mb < LB; ++mb)
                bf[mb] = *reinterpret_cast<const uint4v*>(a_ring + slot * kAStep + static_cast<uint32_t>(mb) * 1024u + b_at);
#pragma unroll
            for (uint32_t t = 0; t < kPfTiles; ++t) {
                uint32_t c0[4], c1[4];
                quad_codewords<WIDE>(wd[0][t], plan, a.wbits, c0);
                quad_codewords<WIDE>(wd[1][t], plan, a.wbits, c1);
                uint4v af;
                af[0] = weight_halves<CB>(c0[0], c0[1]);
                af[1] = weight_halves<CB>(c0[2], c0[3]);
                af[2] = weight_halves<CB>(c1[0], c1[1]);
                af[3] = weight_halves<CB>(c1[2], c1[3]);
#pragma unroll
                for (int mb = 0; mb < LB; ++mb)
                    acc[mb][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        __builtin_bit_cast(half8, af), __builtin_bit_cast(half8, bf[mb]), acc[mb][t], 0, 0, 0);
            }
        };
        // Step s: its operands are in ring slot s % D. The loads of step s + D - 1 go out (into the slot step s - 1
        // left: every wave is past the barrier that ended it), step s + 1's have landed once at most D - 2 steps' loads
        // are in flight, its words are read while step s computes, and the barrier publishes every wave's part of its
        // activations. Loads past the last step fall outside the buffers: they keep the count and bring zeros.
        auto step = [&](uint32_t s, uint32_t slot, const QuadWords<WIDE>(&cur)[2][kPfTiles],
                        QuadWords<WIDE>(&next)[2][kPfTiles]) {
            issue(s + D - 1u, slot == 0u ? D - 1u : slot - 1u);
            wait_loads<static_cast<int>(D - 2u) * kPerStep>();
            fetch_w(next, slot + 1u == D ? 0u : slot + 1u);
            compute(cur, slot);
            __syncthreads();
        };

        QuadWords<WIDE> wd0[2][kPfTiles], wd1[2][kPfTiles];
#pragma unroll
        for (uint32_t t = 0; t + 1u < D; ++t) issue(t, t);
        wait_loads<static_cast<int>(D - 2u) * kPerStep>();
        fetch_w(wd0, 0u);
        __syncthreads();
        uint32_t slot = 0;
        for (uint32_t s = 0; s < steps; s += 2u) {
            step(s, slot, wd0, wd1);
            slot = slot + 1u == D ? 0u : slot + 1u;
            step(s + 1u, slot, wd1, wd0);
            slot = slot + 1u == D ? 0u : slot + 1u;
        }
        wait_loads<0>();

        if (!active) return;
        // D[i][j]: i = the weight's column inside its tile (this lane: 4 (lane / 16) .. + 3), j = activation row
        // lane % 16
#pragma unroll
        for (int mb = 0; mb < LB; ++mb) {
            const uint32_t row = static_cast<uint32_t>(mb) * 16u + (lane & 15u);
            if (row >= count) continue;
            const size_t at = static_cast<size_t>(first + row) * a.out + col0 * 16u + 4u * (lane >> 4);
            if (a.zhalf) {  // uniform
                uint16_t* zh = reinterpret_cast<uint16_t*>(z);
                // the deferred map as the stages apply it to an f32 plane: fma(sum, A, B * total), then the rounding
                const float* xt = a.xtot[proj];
                const float bx = xt ? mul1_b() * xt[first + row] : 0.0f;
#pragma unroll
                for (uint32_t t = 0; t < kPfTiles; ++t) {
                    float4v v = acc[mb][t];
                    if (xt) {
#pragma unroll
                        for (int c = 0; c < 4; ++c) v[c] = __builtin_fmaf(v[c], mul1_a(), bx);
                    }
                    uint2v h;
                    h[0] = static_cast<uint32_t>(half_bits(v[0])) | (static_cast<uint32_t>(half_bits(v[1])) << 16);
                    h[1] = static_cast<uint32_t>(half_bits(v[2])) | (static_cast<uint32_t>(half_bits(v[3])) << 16);
                    *reinterpret_cast<uint2v*>(zh + at + t * 16u) = h;
                }
            } else {
#pragma unroll
                for (uint32_t t = 0; t < kPfTiles; ++t) *reinterpret_cast<float4v*>(z + at + t * 16u) = acc[mb][t];
            }
        }
    };

    const uint32_t live_blocks = (count + 15u) >> 4;  // uniform over the workgroup
    if constexpr (RB == 2) {
        if (live_blocks <= 1u) run.template operator()<1>();
        else run.template operator()<2>();
    } else if constexpr (RB == 4) {
        switch (live_blocks) {
            case 1: run.template operator()<1>(); break;
            case 2: run.template operator()<2>(); break;
            case 3: run.template operator()<3>(); break;
            default: run.template operator()<4>(); break;
        }
    } else if constexpr (kShort) {
        switch (live_blocks) {
            case 1: run.template operator()<1>(); break;
            case 2: run.template operator()<2>(); break;
            case 3: run.template operator()<3>(); break;
            case 4: run.template operator()<4>(); break;
            case 5: run.template operator()<5>(); break;
            default: run.template operator()<6>(); break;
        }
    } else {
        switch (live_blocks) {
            case 1: run.template operator()<1>(); break;
            case 2: run.template operator()<2>(); break;
            case 3: run.template operator()<3>(); break;
            case 4: run.template operator()<4>(); break;
            case 5: run.template operator()<5>(); break;
            case 6: run.template operator()<6>(); break;
            case 7: run.template operator()<7>(); break;
            default: run.template operator()<8>(); break;
        }
    }
}

// ---- the route (src/hip/plan.zig:40-45,412-415: order, inv, items, counts) -------------------------------------

// expert number of a row-slot in [0, experts + shared slots), or ~0 for a skipped id
__device__ __forceinline__ uint32_t slot_expert(const MoeLaunch& a, uint32_t rk) {
    const SlotRef s = resolve_slot(a, rk);
    if (!s.live) return ~0u;
    return s.shared ? a.bank.experts + s.e : s.e;
}

// The experts' counters the row-slots count themselves in at (the histogram, then the placement's cursors) lie a cache
// line apart: side by side, 32 of them share a line and a call's thousands of atomics queue up at a handful of lines
// (81,920 row-slots over 512 experts: the histogram 26 us, the placement 27).
constexpr uint32_t kPfCounterStride = 32u;  // words: 128 bytes

__global__ void __launch_bounds__(256) pf_clear(uint32_t* cursor, uint32_t len) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i < len) cursor[i * kPfCounterStride] = 0u;
}

__global__ void __launch_bounds__(256) pf_hist(const MoeLaunch a) {
    const uint32_t rk = blockIdx.x * 256u + threadIdx.x;
    if (rk >= a.rows * (a.topk + a.shared_slots)) return;
    const uint32_t e = slot_expert(a, rk);
    if (e != ~0u) atomicAdd(a.cursor + e * kPfCounterStride, 1u);
}

// One workgroup of 1024: exclusive sums of the experts' counts (positions) and of their item counts; every expert
// writes its own items. counts[E]: items in all; counts[E + 1]: positions placed.
__global__ void __launch_bounds__(1024) pf_scan(const MoeLaunch a) {
    __shared__ uint32_t wave_pos[16], wave_items[16], carry[2];
    const uint32_t et = a.bank.experts + a.shared_slots, tid = threadIdx.x, lane = tid & 63u, wv = tid >> 6;
    if (tid == 0u) carry[0] = carry[1] = 0u;
    __syncthreads();
    for (uint32_t base = 0; base < et; base += 1024u) {
        const uint32_t e = base + tid;
        const uint32_t c = e < et ? a.cursor[e * kPfCounterStride] : 0u;
        const uint32_t ni = (c + a.item_rows - 1u) / a.item_rows;
        uint32_t pos = c, it = ni;  // inclusive sums inside the wave
#pragma unroll
        for (uint32_t d = 1; d < 64u; d <<= 1) {
            const uint32_t p = __shfl_up(pos, d, 64), q = __shfl_up(it, d, 64);
            if (lane >= d) {
                pos += p;
                it += q;
            }
        }
        if (lane == 63u) {
            wave_pos[wv] = pos;
            wave_items[wv] = it;
        }
        __syncthreads();
        uint32_t pos0 = carry[0], it0 = carry[1];
        for (uint32_t w = 0; w < wv; ++w) {
            pos0 += wave_pos[w];
            it0 += wave_items[w];
        }
        pos0 += pos - c;  // exclusive
        it0 += it - ni;
        if (e < et) {
            a.counts[e] = c;
            a.cursor[e * kPfCounterStride] = pos0;
            for (uint32_t i = 0; i < ni; ++i) {
                uint32_t* item = a.items + static_cast<size_t>(it0 + i) * 4u;
                const uint32_t left = c - i * a.item_rows;
                item[0] = e;
                item[1] = pos0 + i * a.item_rows;
                item[2] = left < a.item_rows ? left : a.item_rows;
                item[3] = 0u;
            }
        }
        __syncthreads();
        if (tid == 1023u) {
            carry[0] = pos0 + c;
            carry[1] = it0 + ni;
        }
        __syncthreads();
    }
    if (tid == 0u) {
        a.counts[et] = carry[1];
        a.counts[et + 1u] = carry[0];
    }
}

// Where a row-slot lands inside its expert's run does not matter to any sum, so the runs are filled in arrival order.
__global__ void __launch_bounds__(256) pf_place(const MoeLaunch a) {
    const uint32_t rk = blockIdx.x * 256u + threadIdx.x;
    if (rk >= a.rows * (a.topk + a.shared_slots)) return;
    const uint32_t e = slot_expert(a, rk);
    if (e == ~0u) {
        a.inv[rk] = ~0u;
        return;
    }
    const uint32_t q = atomicAdd(a.cursor + e * kPfCounterStride, 1u);
    a.order[q] = rk;
    a.inv[rk] = q;
}

// ---- the chains' stages around the GEMM -----------------------------------------------------------------------
// One wave takes kPfUnit adjacent 128-blocks of one row (or sorted position), 16 lanes a block and 8 adjacent elements
// a lane (t3_stages.hpp, "four 128-blocks a wave"): every load and store is 16 bytes a lane, and a block's transform
// is ~20 vector-ALU operations a lane (the one-block-a-wave form of the decode kernels spends ~100: these kernels were
// bound by it). Four waves a workgroup; grid ceil(units / 4). Blocks past the row's last one load the last block and
// store nothing. Every array these kernels touch starts 16-byte aligned (the host checks the caller's).

constexpr uint32_t kPfUnit = 4;

__device__ __forceinline__ uint32_t wave_unit() { return blockIdx.x * 4u + (threadIdx.x >> 6); }

template <int DT, int PROF>
__global__ void __launch_bounds__(256) pf_prep(const MoeLaunch a) {
    const uint32_t nb = a.hidden / 128u, groups = (nb + kPfUnit - 1u) / kPfUnit;
    const uint32_t u0 = wave_unit(), pos = u0 / groups, lane = threadIdx.x & 63u, q = lane & 15u;
    if (pos >= a.counts[a.bank.experts + a.shared_slots + 1u]) return;
    const uint32_t b1 = (u0 % groups) * kPfUnit + (lane >> 4);
    const bool live = b1 < nb;
    const uint32_t b = live ? b1 : nb - 1u, i = b * 128u + 8u * q;
    const SlotRef s = resolve_slot(a, a.order[pos]);
    const RoutedBank& bank = s.shared ? a.shared : a.bank;
    const Row16 g16 = row16(lane);
    float xv[8], sc[2][8];
    load8_act<DT>(a.x, static_cast<size_t>(s.row) * a.hidden + i, xv);
    load8_half(bank.gate_suh, static_cast<size_t>(s.e) * a.hidden + i, sc[0]);
    load8_half(bank.up_suh, static_cast<size_t>(s.e) * a.hidden + i, sc[1]);
#pragma unroll
    for (uint32_t proj = 0; proj < 2u; ++proj) {
        float v[8];
#pragma unroll
        for (uint32_t r = 0; r < 8u; ++r) v[r] = (PROF == 0 ? round_half(xv[r]) : xv[r]) * sc[proj][r];
        uint32_t hv[4];
        float sum;
        prep_row16(v, g16, hv, sum, a.defer != 0);
        if (!live) continue;
        store_pair_quad(reinterpret_cast<uint16_t*>(proj ? a.xu : a.xg), static_cast<size_t>(pos) * a.hidden, b, q, hv);
        if (q == 0u) (proj ? a.su : a.sg)[static_cast<size_t>(pos) * nb + b] = sum;
    }
}

// gate and up finishes, the (clamped) SwiGLU, the down's prepare (routed_mid_block's statements)
// PROF 0: a wave's four blocks are four adjacent (position, block) pairs of all the call's, so that a width that is not
// whole units (640 = five blocks: two units a position, the second a quarter full) wastes no lanes (8192 rows of 512
// experts of 2560 x 640: 185 -> 125 us); a 16-lane group then has a position of its own. GLM's profile adds its block
// sums up across the wave and keeps one position a wave.
template <int PROF>
__global__ void __launch_bounds__(256) pf_mid(const MoeLaunch a) {
    const uint32_t nb = a.inter / 128u, nbh = a.hidden / 128u, groups = (nb + kPfUnit - 1u) / kPfUnit;
    const uint32_t u0 = wave_unit(), lane = threadIdx.x & 63u, q = lane & 15u;
    const uint32_t placed = a.counts[a.bank.experts + a.shared_slots + 1u];
    uint32_t pos, b1;
    bool live;
    if constexpr (PROF == 0) {
        const uint32_t total = placed * nb, f = u0 * kPfUnit + (lane >> 4);
        if (u0 * kPfUnit >= total) return;  // uniform over the wave
        live = f < total;
        const uint32_t fc = live ? f : total - 1u;
        pos = fc / nb;
        b1 = fc - pos * nb;
    } else {
        pos = u0 / groups;
        if (pos >= placed) return;
        b1 = (u0 % groups) * kPfUnit + (lane >> 4);
        live = b1 < nb;
    }
    const uint32_t b = live ? b1 : nb - 1u, i = b * 128u + 8u * q;
    const SlotRef s = resolve_slot(a, a.order[pos]);
    const RoutedBank& bank = s.shared ? a.shared : a.bank;
    const size_t eo = static_cast<size_t>(s.e) * a.inter, qo = static_cast<size_t>(pos) * a.inter;
    const Row16 g16 = row16(lane);
    float gt[8], up[8], svg[8], svu[8], sdn[8];
    const bool zhalf = PROF == 0;  // the GEMM applied the deferred map, if any, before it rounded
    load8_plane(a.zg, qo + i, zhalf, gt);
    load8_plane(a.zu, qo + i, zhalf, up);
    load8_half(bank.gate_svh, eo + i, svg);
    load8_half(bank.up_svh, eo + i, svu);
    load8_half(bank.down_suh, eo + i, sdn);
    if (a.defer && !zhalf) {
        const float xg = wave_ordered_sum(a.sg + static_cast<size_t>(pos) * nbh, nbh, lane);
        const float xu = wave_ordered_sum(a.su + static_cast<size_t>(pos) * nbh, nbh, lane);
#pragma unroll
        for (uint32_t r = 0; r < 8u; ++r) {
            gt[r] = __builtin_fmaf(gt[r], mul1_a(), mul1_b() * xg);
            up[r] = __builtin_fmaf(up[r], mul1_a(), mul1_b() * xu);
        }
    }
    float d[8];
    if constexpr (PROF == 0) {
        finish_row16(gt, svg, g16);
        finish_row16(up, svu, g16);
#pragma unroll
        for (uint32_t r = 0; r < 8u; ++r) d[r] = round_half(swiglu_clamped(gt[r], up[r], a.limit, a.clamp_at)) * sdn[r];
    } else {
        finish_row16_glm(gt, svg, g16, true);
        finish_row16_glm(up, svu, g16, true);
#pragma unroll
        for (uint32_t r = 0; r < 8u; ++r) d[r] = swiglu_glm(gt[r], up[r], a.limit) * sdn[r];
    }
    uint32_t hv[4];
    float sum;
    prep_row16(d, g16, hv, sum, a.defer != 0);
    if (!live) return;
    store_pair_quad(reinterpret_cast<uint16_t*>(a.hd), qo, b, q, hv);
    if (q == 0u) a.hs[static_cast<size_t>(pos) * nb + b] = sum;
}

// GLM's profile: each placed row-slot's down finish as f32 [row-slot][hidden] (routed_slots_block's statements), by
// sorted position
__global__ void __launch_bounds__(256) pf_slots(const MoeLaunch a) {
    const uint32_t nb = a.hidden / 128u, nbi = a.inter / 128u, groups = (nb + kPfUnit - 1u) / kPfUnit;
    const uint32_t u0 = wave_unit(), pos = u0 / groups, lane = threadIdx.x & 63u, q = lane & 15u;
    if (pos >= a.counts[a.bank.experts + a.shared_slots + 1u]) return;
    const uint32_t b1 = (u0 % groups) * kPfUnit + (lane >> 4);
    const bool live = b1 < nb;
    const uint32_t b = live ? b1 : nb - 1u, i = b * 128u + 8u * q;
    const uint32_t rk = a.order[pos];
    const SlotRef s = resolve_slot(a, rk);
    const Row16 g16 = row16(lane);
    float v[8], sv[8];
    load8_f32(a.zd, static_cast<size_t>(pos) * a.hidden + i, v);
    load8_half(a.bank.down_svh, static_cast<size_t>(s.e) * a.hidden + i, sv);
    if (a.defer) {
        const float xsum = wave_ordered_sum(a.hs + static_cast<size_t>(pos) * nbi, nbi, lane);
#pragma unroll
        for (uint32_t r = 0; r < 8u; ++r) v[r] = __builtin_fmaf(v[r], mul1_a(), mul1_b() * xsum);
    }
    finish_row16_glm(v, sv, g16, false);
    if (live) store8_act<kF32>(a.y, static_cast<size_t>(rk) * a.hidden + i, v);
}

// A position's total of its input's block sums, 0 + s[0] + s[1] + ... (wave_ordered_sum's order): what MUL1's deferred map
// multiplies by B. Made once a position here so that the GEMM's end can apply the map to its sums and round them (f16
// planes: the stages after it read half the bytes). A thread a position; up to two arrays a launch.
__global__ void __launch_bounds__(256) pf_rowsums(const float* s0, const float* s1, float* t0, float* t1, uint32_t nb,
                                                  uint32_t positions) {
    const uint32_t pos = blockIdx.x * 256u + threadIdx.x;
    if (pos >= positions) return;
    const float* s = blockIdx.y ? s1 : s0;
    float acc = 0.0f;
    for (uint32_t b = 0; b < nb; ++b) acc += s[static_cast<size_t>(pos) * nb + b];
    (blockIdx.y ? t1 : t0)[pos] = acc;
}

// every slot's down finish, then the score-weighted sum in slot order (routed_combine_block's statements)
__global__ void __launch_bounds__(256) pf_combine(const MoeLaunch a) {
    const uint32_t nb = a.hidden / 128u, groups = (nb + kPfUnit - 1u) / kPfUnit;
    const uint32_t u0 = wave_unit(), row = u0 / groups, lane = threadIdx.x & 63u, q = lane & 15u;
    if (row >= a.rows) return;
    const uint32_t b1 = (u0 % groups) * kPfUnit + (lane >> 4);
    const bool live = b1 < nb;
    const uint32_t b = live ? b1 : nb - 1u, i = b * 128u + 8u * q;
    const Row16 g16 = row16(lane);
    const uint32_t kt = a.topk + a.shared_slots;
    float acc[8];
#pragma unroll
    for (uint32_t r = 0; r < 8u; ++r) acc[r] = 0.0f;
    for (uint32_t k = 0; k < kt; ++k) {
        const uint32_t rk = row * kt + k;
        const SlotRef s = resolve_slot(a, rk);
        if (!s.live) continue;  // uniform over the wave
        const uint32_t pos = a.inv[rk];
        const RoutedBank& bank = s.shared ? a.shared : a.bank;
        float v[8], sv[8];
        // f16: the down GEMM applied the deferred map, if any, before it rounded
        load8_plane(a.zd, static_cast<size_t>(pos) * a.hidden + i, true, v);
        load8_half(bank.down_svh, static_cast<size_t>(s.e) * a.hidden + i, sv);
        const float w = s.shared ? 1.0f : score_of(a, row, k);
        finish_row16(v, sv, g16);
#pragma unroll
        for (uint32_t r = 0; r < 8u; ++r) acc[r] = __builtin_fmaf(w, v[r], acc[r]);
    }
    if (!live) return;
    const size_t o = static_cast<size_t>(row) * a.hidden + i;
    if (a.shared_add) {
        // the routed output rounds to x's dtype, then the add rounds again (src/root.zig:976-984)
        float add[8];
        load8_act_rt(a.dtype, a.shared_add, o, add);
#pragma unroll
        for (uint32_t r = 0; r < 8u; ++r) {
            float t = acc[r];
            if (a.dtype == kF16) t = round_half(t);
            else if (a.dtype == kBf16) t = bf16_value(bf16_bits(t));
            acc[r] = t + add[r];
        }
    }
    store8_act_rt(a.dtype, a.y, o, acc);
}

// the dense prepare: plain f16 [rows][in], in pair-quad order for the trellis GEMM (NATURAL: as is, for a plain GEMM);
// xs: block sums (null: not wanted)
template <int DT, bool NATURAL>
__global__ void __launch_bounds__(256) pf_dense_prep(const void* x, const uint16_t* suh, uint16_t* xq, float* xs,
                                                     uint32_t in, uint32_t rows) {
    const uint32_t nb = in / 128u, groups = (nb + kPfUnit - 1u) / kPfUnit;
    const uint32_t u0 = wave_unit(), row = u0 / groups, lane = threadIdx.x & 63u, q = lane & 15u;
    if (row >= rows) return;
    const uint32_t b1 = (u0 % groups) * kPfUnit + (lane >> 4);
    const bool live = b1 < nb;
    const uint32_t b = live ? b1 : nb - 1u, i = b * 128u + 8u * q;
    const Row16 g16 = row16(lane);
    float v[8], sc[8];
    load8_act<DT>(x, static_cast<size_t>(row) * in + i, v);
    load8_half(suh, i, sc);
#pragma unroll
    for (uint32_t r = 0; r < 8u; ++r) v[r] = round_half(v[r]) * sc[r];
    uint32_t hv[4];
    float sum;
    prep_row16(v, g16, hv, sum, xs != nullptr);
    if (!live) return;
    if constexpr (NATURAL)
        *reinterpret_cast<uint4v*>(xq + static_cast<size_t>(row) * in + i) = uint4v{hv[0], hv[1], hv[2], hv[3]};
    else
        store_pair_quad(xq, static_cast<size_t>(row) * in, b, q, hv);
    if (xs && q == 0u) xs[static_cast<size_t>(row) * nb + b] = sum;
}

// the dense finish: z f32 [ks][rows][out], the planes summed in part order, with xs [rows][in / 128] for MUL1's deferred
// map
template <int DT>
__global__ void __launch_bounds__(256) pf_dense_finish(const float* z, const float* xs, const uint16_t* svh, void* y,
                                                       uint32_t out, uint32_t rows, uint32_t inblk, int defer,
                                                       uint32_t ks) {
    const uint32_t nb = out / 128u, groups = (nb + kPfUnit - 1u) / kPfUnit;
    const uint32_t u0 = wave_unit(), row = u0 / groups, lane = threadIdx.x & 63u, q = lane & 15u;
    if (row >= rows) return;
    const uint32_t b1 = (u0 % groups) * kPfUnit + (lane >> 4);
    const bool live = b1 < nb;
    const uint32_t b = live ? b1 : nb - 1u, i = b * 128u + 8u * q;
    const Row16 g16 = row16(lane);
    const size_t at = static_cast<size_t>(row) * out + i;
    float v[8], sv[8];
    load8_plane(z, at, ks == 1u && !defer, v);
    const size_t plane = static_cast<size_t>(rows) * out;
    for (uint32_t k = 1; k < ks; ++k) {
        float part[8];
        load8_f32(z + k * plane, at, part);
#pragma unroll
        for (uint32_t r = 0; r < 8u; ++r) v[r] += part[r];
    }
    load8_half(svh, i, sv);
    if (defer) {
        const float xsum = wave_ordered_sum(xs + static_cast<size_t>(row) * inblk, inblk, lane);
#pragma unroll
        for (uint32_t r = 0; r < 8u; ++r) v[r] = __builtin_fmaf(v[r], mul1_a(), mul1_b() * xsum);
    }
    finish_row16(v, sv, g16);
    if (live) store8_act<DT>(y, at, v);
}

inline dim3 unit_grid(uint32_t rows, uint32_t width) {
    const uint32_t groups = (width / 128u + kPfUnit - 1u) / kPfUnit;
    return dim3((rows * groups + 3u) / 4u);
}

template <bool NATURAL>
hipError_t launch_pf_dense_prep(const DenseLaunch& d, uint16_t* xq, float* xs, hipStream_t s) {
    const dim3 grid = unit_grid(d.rows, d.in), block(256);
    if (d.dtype == kF32) hipLaunchKernelGGL((pf_dense_prep<kF32, NATURAL>), grid, block, 0, s, d.x, d.suh, xq, xs, d.in, d.rows);
    else if (d.dtype == kF16) hipLaunchKernelGGL((pf_dense_prep<kF16, NATURAL>), grid, block, 0, s, d.x, d.suh, xq, xs, d.in, d.rows);
    else hipLaunchKernelGGL((pf_dense_prep<kBf16, NATURAL>), grid, block, 0, s, d.x, d.suh, xq, xs, d.in, d.rows);
    return hipGetLastError();
}

hipError_t launch_pf_dense_finish(const DenseLaunch& d, const float* z, hipStream_t s) {
    const dim3 grid = unit_grid(d.rows, d.out), block(256);
    const uint32_t inblk = d.in / 128u;
    const int defer = d.codebook == kMul1Defer ? 1 : 0;
    if (d.dtype == kF32) hipLaunchKernelGGL(pf_dense_finish<kF32>, grid, block, 0, s, z, d.xs, d.svh, d.y, d.out, d.rows, inblk, defer, d.ks);
    else if (d.dtype == kF16) hipLaunchKernelGGL(pf_dense_finish<kF16>, grid, block, 0, s, z, d.xs, d.svh, d.y, d.out, d.rows, inblk, defer, d.ks);
    else hipLaunchKernelGGL(pf_dense_finish<kBf16>, grid, block, 0, s, z, d.xs, d.svh, d.y, d.out, d.rows, inblk, defer, d.ks);
    return hipGetLastError();
}

// workgroup columns of a GEMM over `out` columns with `item_rows`-row items
inline uint32_t gemm_nblk(uint32_t out, uint32_t item_rows) {
    (void)item_rows;
    return (out + 255u) / 256u;
}

template <int CB, int WIDE>
hipError_t launch_gemm_rb(PfGemm g, uint32_t max_items, uint32_t nproj, uint32_t item_rows, hipStream_t s) {
    g.nblk = gemm_nblk(g.out, item_rows);
    g.spread = gemm_spread(max_items);  // 8 / spread items share the dies
    if (g.kparts == 0u) g.kparts = 1u;
    const dim3 grid(gemm_grid_x(g.nblk, max_items), nproj, g.kparts), block(256);
    if (item_rows == 32u) hipLaunchKernelGGL((pf_gemm<CB, WIDE, 2>), grid, block, 0, s, g);
    else if (item_rows == 128u) hipLaunchKernelGGL((pf_gemm<CB, WIDE, 8>), grid, block, 0, s, g);
    else if (item_rows == 96u) hipLaunchKernelGGL((pf_gemm<CB, WIDE, 8, 6>), grid, block, 0, s, g);
    else hipLaunchKernelGGL((pf_gemm<CB, WIDE, 4>), grid, block, 0, s, g);
    return hipGetLastError();
}

// The GEMM decodes exactly whatever form the GEMV runs: MCG's pair form has no use here (it would double K).
hipError_t launch_gemm(const PfGemm& g, int codebook, uint32_t max_items, uint32_t nproj, uint32_t item_rows,
                       hipStream_t s) {
    return with_reader(g.n, [&](auto reader) {
        constexpr int R = decltype(reader)::value;
        switch (codebook) {
            case kMul1: return launch_gemm_rb<kMul1, R>(g, max_items, nproj, item_rows, s);
            case kMul1Defer: return launch_gemm_rb<kMul1Defer, R>(g, max_items, nproj, item_rows, s);
            default: return launch_gemm_rb<kMcg, R>(g, max_items, nproj, item_rows, s);
        }
    });
}

}  // namespace

hipError_t launch_moe_prefill(const MoeLaunch& a, hipStream_t s) {
    const uint32_t kt = a.topk + a.shared_slots, p = a.rows * kt, et = a.bank.experts + a.shared_slots;
    hipError_t e;
    if (a.stages & 1u) {
        hipLaunchKernelGGL(pf_clear, dim3((et + 255u) / 256u), dim3(256), 0, s, a.cursor, et);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        hipLaunchKernelGGL(pf_hist, dim3((p + 255u) / 256u), dim3(256), 0, s, a);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        hipLaunchKernelGGL(pf_scan, dim3(1), dim3(1024), 0, s, a);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        hipLaunchKernelGGL(pf_place, dim3((p + 255u) / 256u), dim3(256), 0, s, a);
        if ((e = hipGetLastError()) != hipSuccess) return e;
    }
    if (a.stages & 2u) {
        if (a.glm) hipLaunchKernelGGL((pf_prep<kBf16, 1>), unit_grid(p, a.hidden), dim3(256), 0, s, a);
        else if (a.dtype == kF32) hipLaunchKernelGGL((pf_prep<kF32, 0>), unit_grid(p, a.hidden), dim3(256), 0, s, a);
        else if (a.dtype == kF16) hipLaunchKernelGGL((pf_prep<kF16, 0>), unit_grid(p, a.hidden), dim3(256), 0, s, a);
        else hipLaunchKernelGGL((pf_prep<kBf16, 0>), unit_grid(p, a.hidden), dim3(256), 0, s, a);
        if ((e = hipGetLastError()) != hipSuccess) return e;
    }

    PfGemm g{};
    g.w[0] = a.bank.gate_t;
    g.w[1] = a.bank.up_t;
    g.ws[0] = a.shared.gate_t;
    g.ws[1] = a.shared.up_t;
    g.xq[0] = reinterpret_cast<const uint16_t*>(a.xg);
    g.xq[1] = reinterpret_cast<const uint16_t*>(a.xu);
    g.z[0] = a.zg;
    g.z[1] = a.zu;
    g.items = a.items;
    g.n_items = a.counts + et;
    g.in = a.hidden;
    g.out = a.inter;
    g.n = a.n_gu;
    g.wbits = a.wbits;
    g.positions = p;
    g.experts = a.bank.experts;
    g.zhalf = !a.glm;
    const bool map = a.defer && !a.glm;  // the GEMMs' ends apply the deferred map (GLM's profile keeps f32 planes)
    g.xtot[0] = map ? a.xt : nullptr;
    g.xtot[1] = map ? a.xt + p : nullptr;
    if (a.stages & 4u) {
        if (map) {
            hipLaunchKernelGGL(pf_rowsums, dim3((p + 255u) / 256u, 2u), dim3(256), 0, s, a.sg, a.su, a.xt, a.xt + p,
                               a.hidden / 128u, p);
            if ((e = hipGetLastError()) != hipSuccess) return e;
        }
        if ((e = launch_gemm(g, a.codebook, a.max_items, 2u, a.item_rows, s)) != hipSuccess) return e;
    }

    if (a.stages & 8u) {
        if (a.glm) hipLaunchKernelGGL(pf_mid<1>, unit_grid(p, a.inter), dim3(256), 0, s, a);
        else hipLaunchKernelGGL(pf_mid<0>, dim3((p * (a.inter / 128u) + 4u * kPfUnit - 1u) / (4u * kPfUnit)), dim3(256), 0, s, a);
        if ((e = hipGetLastError()) != hipSuccess) return e;
    }

    g.w[0] = a.bank.down_t;
    g.ws[0] = a.shared.down_t;
    g.w[1] = g.ws[1] = nullptr;
    g.xq[0] = reinterpret_cast<const uint16_t*>(a.hd);
    g.xq[1] = nullptr;
    g.z[0] = a.zd;
    g.z[1] = nullptr;
    g.in = a.inter;
    g.out = a.hidden;
    g.n = a.n_dn;
    g.xtot[0] = map ? a.xt + 2u * static_cast<size_t>(p) : nullptr;
    g.xtot[1] = nullptr;
    if (a.stages & 16u) {
        if (map) {
            hipLaunchKernelGGL(pf_rowsums, dim3((p + 255u) / 256u, 1u), dim3(256), 0, s, a.hs, a.hs, a.xt + 2u * static_cast<size_t>(p),
                               a.xt + 2u * static_cast<size_t>(p), a.inter / 128u, p);
            if ((e = hipGetLastError()) != hipSuccess) return e;
        }
        if ((e = launch_gemm(g, a.codebook, a.max_items, 1u, a.item_rows, s)) != hipSuccess) return e;
    }

    if (!(a.stages & 32u)) return hipSuccess;
    if (a.glm) hipLaunchKernelGGL(pf_slots, unit_grid(p, a.hidden), dim3(256), 0, s, a);
    else hipLaunchKernelGGL(pf_combine, unit_grid(a.rows, a.hidden), dim3(256), 0, s, a);
    return hipGetLastError();
}

hipError_t launch_dense_planes_finish(const DenseLaunch& d, const float* planes, uint32_t kparts, hipStream_t s) {
    DenseLaunch f = d;
    f.ks = kparts;
    f.codebook = kMcg;  // finished weights went into the product: no deferred map
    return launch_pf_dense_finish(f, planes, s);
}

hipError_t launch_dense_prep_natural(const DenseLaunch& d, uint16_t* xp, hipStream_t s) {
    return launch_pf_dense_prep<true>(d, xp, nullptr, s);
}

hipError_t launch_dense_prefill(const DenseLaunch& d, hipStream_t s) {
    hipError_t e;
    // the block sums feed MUL1's deferred map only
    float* xs = d.codebook == kMul1Defer ? d.xs : nullptr;
    if ((e = launch_pf_dense_prep<false>(d, reinterpret_cast<uint16_t*>(d.xq), xs, s)) != hipSuccess) return e;
    PfGemm g{};
    g.w[0] = d.trellis;
    g.xq[0] = reinterpret_cast<const uint16_t*>(d.xq);
    g.z[0] = d.z;
    g.in = d.in;
    g.out = d.out;
    g.n = d.n;
    g.wbits = d.wbits;
    g.positions = d.rows;
    g.experts = 1u;
    g.kparts = d.ks;
    g.plane = d.rows * d.out;
    g.zhalf = d.ks == 1u && d.codebook != kMul1Defer;
    const uint32_t item_rows = d.rows <= 64u ? 64u : 128u;
    if ((e = launch_gemm(g, d.codebook, (d.rows + item_rows - 1u) / item_rows, 1u, item_rows, s)) != hipSuccess) return e;
    return launch_pf_dense_finish(d, d.z, s);
}

}  // namespace t3
