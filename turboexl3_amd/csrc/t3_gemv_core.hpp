// The streaming core every decode-row GEMV of this library runs: one wave walks `per` tile rows of a trellis matrix
// (BT adjacent 16x16 tiles a row), decodes each tile a quad of weights a lane straight into the A fragment of
// v_mfma_f32_16x16x32_f16, and multiplies by up to 32 prepared activation rows held as B fragments.
//
// Memory path. A tile row's BT tiles are contiguous (BT * 2n bytes <= 1 KB), so a wave fetches them with ONE 128-bit
// buffer load, 16 consecutive bytes a lane: the texture unit sees a fully coalesced stream (a gather of each lane's
// own words costs it many times the cycles, measured). The bytes pass through a wave-private piece of LDS, one slot a
// tile, and every lane reads back the two words its quad needs (four at the wide rates whose quads pass two words).
// Two forms of the way into LDS, the same sums either way (a lane decodes the same words in the same order):
//   GemvStreamRegs  global -> a ring of two loads in registers -> ds_write -> LDS (two stage buffers) -> registers;
//   GemvStreamLds   global -> LDS directly (buffer_load_dwordx4 ... lds: lane L's 16 bytes land at M0 + 16 L), a ring of
//                   four tile rows' slots a wave, three rows in flight under a decode, no staging registers, no
//                   ds_write. The loads are issued from inline asm, so the compiler neither sees nor waits for them:
//                   the stream counts them itself (s_waitcnt vmcnt(N); a wave's vector-memory operations complete in
//                   order, so whatever else the wave has in that queue only makes a wait longer).
// Measured on one box (us; register ring / LDS ring of four / LDS ring of eight): one row of 4096 x 12288 K4, the call
// 15.3 / 15.6 / 16.8, 16 rows 20.2 / 20.5 / 20.9, 32 rows 24.1 / 24.8 / 29.6; one row of 4096 x 151936 (the GEMV launch)
// K3 102 / 98 / 98, K4 103 / 100 / 99, K5 109 / 103 / 108, K6 118 / 111 / 125; the routed call at one and eight tokens
// 25.9 / 25.1 / 25.5 and 65.5 / 64.4 / 69: the LDS ring pays where a wave's walk is long (the deeper ring's LDS costs
// occupancy), and a launch of a few tile rows a wave starts sooner with two rows requested a wave than with four.
// The host serves the LDS ring from 32 tile rows a wave (dense_gemv_lds_ring), the register ring below.
//
// The prepared activations are B fragments as they lie in memory, 16 bytes a lane (XGlobal: ordinary loads into a
// register ring beside the tiles'; through LDS they cost a 1 KB write and read a tile row for 64 useful bytes a row,
// measured at 16 rows: 20.3 -> 21.7 us a call; loaded from asm into registers, the compiler moves them across the loop's
// back edge before they have landed), or are made in LDS by the wave itself (XLds).
// A row past the wave's last is read through a zero-sized buffer: zeros, no memory is touched.
//
// Steps. The forms that feed the matrix core a weight in a PAIR of K slots (MCG's hashed pair; MUL1's h with its deferred
// map, whose packing of two weights a register would cost the instruction it saves) take one tile row a step: a lane's
// quad fills the fragment's eight K slots. The forms that feed the format's f16 weight take TWO tile rows a step: eight
// different weights a lane (the quad of tile row 2s in K slots 0..3, of 2s + 1 in 4..7; the sub-dword add and
// multiply-add that round a weight write either half of a register, so the packing is free), against activations kept in
// "pair-quad order" (plain f16: inside every 32 inputs, quad q of the first tile row then quad q of the second), so a
// tile costs half an MFMA.
//
// Sums: each MFMA output element depends on its own activation row alone, and a wave's tile rows are taken in
// ascending order, so a row's partial sum is a function of (matrix, K part, row) only.
//
// Cost model (measured on MI355X): per tile a lane issues 13 vector-ALU instructions in the pair and deferred forms
// (1 v_alignbit, then v_bfe, v_mul_lo, v_bitop3 a weight; 17 with the f16 add of MCG's exact weight), 4 cycles of a
// SIMD's issue each, and one MFMA, about half of whose 16 cycles overlap other waves' vector-ALU work: the kernel is
// instruction-bound below 6 bits a weight.
#pragma once

#include <type_traits>

#include "t3_decode.hpp"
#include "t3_lds_loads.hpp"

namespace t3 {

constexpr uint32_t kTileSlot = 256u;  // register ring: LDS bytes a staged tile (2n <= 256)
// Activation rows the in-LDS form of the prepared input holds. (A build-time override for measuring the one-launch dense
// form at more rows, with T3_ONE_ROWS_BT8 of t3_linear.cpp: 16 rows took 23.3 us a call against the chain's 18.1 at
// 4096 x 12288 K4: every column workgroup prepares every row of its K part again.)
#ifndef T3_XLDS_ROWS
#define T3_XLDS_ROWS 4u
#endif
constexpr uint32_t kXldsRows = T3_XLDS_ROWS;
constexpr uint32_t kRowSlot = 1024u;  // LDS ring: bytes one load of a wave fills: 64 lanes x 16 bytes
constexpr uint32_t kNoBytes = 0x80000000u;  // a lane offset no buffer reaches: zeros, no traffic

// tile rows a step of codebook form CB
template <int CB>
constexpr int gemv_step_rows() {
    return (CB == kMcg || CB == kMul1 || CB == kMcgTab) ? 2 : 1;
}

// Where a wave's prepared activations come from. A step's activations are 64 bytes a row either way: 16 inputs doubled
// (one tile row a step), or 32 inputs as plain f16 in pair-quad order (two).
struct XGlobal {
    const uint32_t* base;
    uint64_t bytes;
    uint32_t first;         // byte offset of the wave's first step
    uint32_t step;          // bytes from one step to the next: 64 where a row's steps are adjacent ([rows][in]),
                            // rows x 64 where a step's rows are ([steps][rows][64 bytes]: the fragment of one step is one
                            // contiguous piece, whole cache lines whatever the rows)
};
struct XLds {               // the wave's own [steps + 1][kXldsRows][64 bytes], written by the in-kernel prepare;
    const unsigned char* base;  // the last step all zeros: what a step past the wave's last multiplies by
};
// Where the in-kernel prepare puts element e (0 .. 16 R - 1) of a step's inputs inside an activation row's 64 bytes
// (byte offset), and whether as a doubled f16 (R = 1: 4 bytes) or a plain one (R = 2: 2 bytes)
template <int R>
__device__ __forceinline__ uint32_t x_step_slot_bytes(uint32_t e) {
    if constexpr (R == 1) return quad_slot(e & 15u) * 4u;
    else return (pair_quad_slot(e) & 31u) * 2u;
}
template <int R>
__device__ __forceinline__ void x_step_store(unsigned char* row64, uint32_t e, uint32_t hbits) {
    if constexpr (R == 1) *reinterpret_cast<uint32_t*>(row64 + x_step_slot_bytes<1>(e)) = hbits | (hbits << 16);
    else *reinterpret_cast<uint16_t*>(row64 + x_step_slot_bytes<2>(e)) = static_cast<uint16_t>(hbits);
}

// XGlobal: the byte offset, inside one step's activations, of a lane's piece of a B fragment: activation row
// lane % 16 of the block lies `row_bytes` into them, the lane's eight K slots are its 16-byte piece lane / 16
// (kNoBytes: that fragment row stays zero).
__device__ __forceinline__ uint32_t x_frag_offset(uint32_t lane, bool live, uint32_t row_bytes) {
    return live ? row_bytes + (lane >> 4) * 16u : kNoBytes;
}

// One wave's stream over `per` tile rows (a multiple of the step's rows), either form. Construct, `issue()` the first
// loads, do whatever else the kernel has to do while they fly (the one-launch form prepares its activations there), then
// `run()`.
//
// wbase: the wave's first tile row (tile 0 of its BT); wstep: bytes from one tile row to the next; per: tile rows.
// xoff[r]: XGlobal: x_frag_offset of block r's fragment; XLds: the lane's byte offset of block r's activation row plus
// its piece inside a step's kXldsRows x 64 bytes. stage: the wave's own LDS bytes (kStageBytes), 16-byte aligned.
// run(): acc[r][t] += the 16 x 16 product of activation block r and tile t, summed over the wave's tile rows in order;
// when it returns none of the wave's loads is in flight and the stage's memory is free.

#ifndef T3_GEMV_TABLE_PAIRS
#define T3_GEMV_TABLE_PAIRS 2
#endif

// What both forms share: a step's words out of its LDS slots, and its decode into the matrix core.
template <int CB, int WIDE, int RB, int BT>
struct GemvStep {
    static constexpr int R = gemv_step_rows<CB>();
    QuadWords<WIDE> wd[R][BT];

    // rows: the step's tile rows in LDS, `row_bytes` apart, a tile's slot `slot_bytes`
    __device__ __forceinline__ void fetch(const unsigned char* rows, uint32_t row_bytes, uint32_t slot_bytes,
                                          const QuadPlan<WIDE>& plan) {
        const uint32_t get_bp = plan.ib_prev * 4u, get_bl = plan.ib_last * 4u;
        const uint32_t get_ap = plan.ia_prev * 4u, get_al = plan.ia_last * 4u;
#pragma unroll
        for (int j = 0; j < R; ++j)
#pragma unroll
            for (int t = 0; t < BT; ++t) {
                const unsigned char* tile = rows + static_cast<uint32_t>(j) * row_bytes + static_cast<uint32_t>(t) * slot_bytes;
                wd[j][t].b_prev = *reinterpret_cast<const uint32_t*>(tile + get_bp);
                wd[j][t].b_last = *reinterpret_cast<const uint32_t*>(tile + get_bl);
                if constexpr (WIDE == kWide) {
                    wd[j][t].a_prev = *reinterpret_cast<const uint32_t*>(tile + get_ap);
                    wd[j][t].a_last = *reinterpret_cast<const uint32_t*>(tile + get_al);
                }
            }
    }
    __device__ __forceinline__ void consume(const QuadPlan<WIDE>& plan, uint32_t wbits, const uint4v (&xv)[RB],
                                            float4v (&acc)[RB][BT]) const {
#pragma unroll
        for (int t = 0; t < BT; ++t) {
            uint4v a;
            if constexpr (R == 1) {
                uint32_t cw[4];
                quad_codewords<WIDE>(wd[0][t], plan, wbits, cw);
#pragma unroll
                for (int m = 0; m < 4; ++m) a[m] = weight_pair<CB>(cw[m]);
            } else {
                uint32_t c0[4], c1[4];
                quad_codewords<WIDE>(wd[0][t], plan, wbits, c0);
                quad_codewords<WIDE>(wd[1][t], plan, wbits, c1);
                if constexpr (CB == kMcgTab) {
                    // T3_GEMV_TABLE_PAIRS of a lane's four registers a tile pair come out of the LDS table, the others
                    // out of the ALU hash: both pipes at work
                    a[0] = T3_GEMV_TABLE_PAIRS >= 1 ? table_halves(c0[0], c0[1]) : weight_halves<kMcg>(c0[0], c0[1]);
                    a[1] = T3_GEMV_TABLE_PAIRS >= 3 ? table_halves(c0[2], c0[3]) : weight_halves<kMcg>(c0[2], c0[3]);
                    a[2] = T3_GEMV_TABLE_PAIRS >= 2 ? table_halves(c1[0], c1[1]) : weight_halves<kMcg>(c1[0], c1[1]);
                    a[3] = T3_GEMV_TABLE_PAIRS >= 4 ? table_halves(c1[2], c1[3]) : weight_halves<kMcg>(c1[2], c1[3]);
                } else {
                    a[0] = weight_halves<CB>(c0[0], c0[1]);
                    a[1] = weight_halves<CB>(c0[2], c0[3]);
                    a[2] = weight_halves<CB>(c1[0], c1[1]);
                    a[3] = weight_halves<CB>(c1[2], c1[3]);
                }
            }
#pragma unroll
            for (int r = 0; r < RB; ++r)
                acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a),
                                                                   __builtin_bit_cast(half8, xv[r]), acc[r][t], 0, 0, 0);
        }
    }
};

template <int CB, int WIDE, int RB, int BT, typename XSrc>
struct GemvStreamRegs {
    static constexpr int R = gemv_step_rows<CB>();   // tile rows a step
#ifndef T3_GEMV_REGS_ST2
#define T3_GEMV_REGS_ST2 1
#endif
    // steps in flight in the register ring: two tile rows' loads a wave either way. (With four requested a wave at its
    // start, a launch of a few tile rows a wave begins later: the same call measured 0.4 us longer.)
    static constexpr int ST = R == 1 ? 2 : T3_GEMV_REGS_ST2;
    // One tile row a step: the words of step s + 1 are read into a second register set while step s decodes, through
    // two stage buffers. Two tile rows a step: one set of words, read when their step begins, and one stage buffer (a
    // wave's LDS operations complete in order: the next step's store follows this step's reads), or the registers and
    // LDS of twice the tiles would cost the kernel a wave of occupancy.
    static constexpr bool kAhead = R == 1;
    static constexpr uint32_t kBufs = kAhead ? 2u : 1u;
    static constexpr uint32_t kBuf = static_cast<uint32_t>(R) * BT * kTileSlot;   // LDS bytes a staged step
    // LDS bytes one wave's stage takes: the buffers, then a dump where the lanes past a tile row's last byte put their
    // (zero) registers, so the store needs neither a branch nor a per-lane buffer offset: 512 bytes, plus what a store to
    // the last buffer adds to every lane's offset alike
    static constexpr uint32_t kStageBytes = kBufs * kBuf + 512u + (kBufs - 1u) * kBuf + static_cast<uint32_t>(R - 1) * BT * kTileSlot;
    static constexpr bool kXLds = __is_same(XSrc, XLds);
    static_assert(!kAhead || ST % 2 == 0, "stage buffers and word sets alternate by ring slot parity");

    const uint32_t* wbase;
    uint32_t wstep, steps, n, wbits, lane;
    XSrc xs;
    uint32_t xoff[RB];
    unsigned char* stage;
    uint32_t span_bytes, voff;
    // Three overlapped pipelines, all in the wave's own program order:
    //   global -> registers   ST steps ahead (ring), the activations beside them: the load counter retires in
    //                         order, so a load issued later than a step's would hold that step's wait back to its lead;
    //   registers -> LDS -> registers   one step ahead (one tile row a step), or as the step begins (two);
    //   decode + MFMA         the step whose words are in registers.
    uint4v ring[ST][R];
    uint4v xr[ST][RB];

    __device__ __forceinline__ GemvStreamRegs(const uint32_t* wbase_, uint32_t wstep_, uint32_t per_, uint32_t n_,
                                              uint32_t wbits_, const XSrc& xs_, const uint32_t (&xoff_)[RB],
                                              unsigned char* stage_, uint32_t lane_)
        : wbase(wbase_), wstep(wstep_), steps(per_ / static_cast<uint32_t>(R)), n(n_), wbits(wbits_), lane(lane_), xs(xs_),
          stage(stage_) {
#pragma unroll
        for (int r = 0; r < RB; ++r) xoff[r] = xoff_[r];
        const uint32_t chunk_bytes = static_cast<uint32_t>(BT) * 2u * n;  // a multiple of 16: BT is 4 or 8, n even
        // bytes from the wave's first tile row to the end of its last (the range check covers the scalar offset too)
        span_bytes = (per_ - 1u) * wstep + chunk_bytes;
        // a lane past the chunk asks for an offset no buffer reaches: zeros, no traffic
        voff = lane * 16u < chunk_bytes ? lane * 16u : kNoBytes;
    }

    __device__ __forceinline__ void load_step(uint32_t step, uint4v (&dst)[R]) const {
        const __amdgpu_buffer_rsrc_t res = make_rsrc(wbase, step < steps ? span_bytes : 0u);
#pragma unroll
        for (int j = 0; j < R; ++j) dst[j] = buf_load_u128(res, voff, (step * R + static_cast<uint32_t>(j)) * wstep);
    }
    __device__ __forceinline__ void load_x(uint32_t step, uint4v (&dst)[RB]) const {
        if constexpr (!kXLds) {
            const __amdgpu_buffer_rsrc_t res = make_rsrc(xs.base, step < steps ? xs.bytes : 0u);
            const uint32_t soff = xs.first + step * xs.step;
#pragma unroll
            for (int r = 0; r < RB; ++r) dst[r] = buf_load_u128(res, xoff[r], soff);
        }
    }

    __device__ __forceinline__ void issue() {
#pragma unroll
        for (int s = 0; s < ST; ++s) {
            load_step(static_cast<uint32_t>(s), ring[s]);
            load_x(static_cast<uint32_t>(s), xr[s]);
            __builtin_amdgcn_sched_barrier(0);  // issue order = ring order: the first step's wait must not cover the rest
        }
    }

    // A tile of whole 16-byte pieces (n a multiple of 8: every standard rate) takes a lane's load into the stage with one
    // 128-bit store; otherwise a lane's four dwords may lie in two tiles and go one by one (four stores at a stride of
    // four banks: each a four-way bank conflict, which the wide rates' LDS traffic has no room for). Two copies of the
    // loop rather than a branch inside it.
    __device__ __forceinline__ void run(float4v (&acc)[RB][BT]) {
        if ((n & 7u) == 0u) run_as<true>(acc);
        else run_as<false>(acc);
    }

    template <bool W16>
    __device__ __forceinline__ void run_as(float4v (&acc)[RB][BT]) {
        const uint32_t tile_bytes = 2u * n;
        const uint32_t chunk_bytes = static_cast<uint32_t>(BT) * tile_bytes;
        // The loads are in flight; everything a lane needs to decode is worked out under their latency.
        const QuadPlan<WIDE> plan = quad_plan<WIDE>(n, lane);
        // where the lane's four loaded dwords land: tile slot + offset inside the tile (a lane past the chunk stores
        // into the dump behind the buffers); b / tile_bytes by a 16-bit reciprocal, exact for b < 1024 and
        // tile_bytes >= 32
        const bool writer = lane * 16u < chunk_bytes;
        const uint32_t inv_tile = (1u << 16) / tile_bytes + 1u;
        uint32_t put[4];
#pragma unroll
        for (uint32_t j = 0; j < 4u; ++j) {
            const uint32_t b = lane * 16u + 4u * j;
            const uint32_t t = (b * inv_tile) >> 16;
            put[j] = writer ? t * kTileSlot + (b - t * tile_bytes) : kBufs * kBuf + (lane & 31u) * 16u + 4u * j;
        }
        // a step's loaded tile rows into stage buffer `buf`
        auto stage_step = [&](const uint4v (&v)[R], uint32_t buf) {
#pragma unroll
            for (int j = 0; j < R; ++j) {
                unsigned char* row = stage + buf * kBuf + static_cast<uint32_t>(j) * (BT * kTileSlot);
                if constexpr (W16) {
                    *reinterpret_cast<uint4v*>(row + put[0]) = v[j];
                } else {
#pragma unroll
                    for (uint32_t k = 0; k < 4u; ++k) *reinterpret_cast<uint32_t*>(row + put[k]) = v[j][k];
                }
            }
        };
        // the LDS form's activations of a step (past the last: the zero step)
        auto fetch_x = [&](uint32_t step, uint4v(&xv)[RB]) {
            if constexpr (kXLds) {
                const uint32_t at = step < steps ? step : steps;
#pragma unroll
                for (int r = 0; r < RB; ++r)
                    xv[r] = *reinterpret_cast<const uint4v*>(xs.base + at * (kXldsRows * 64u) + xoff[r]);
            }
        };

        // No branch inside the ring: a step past the wave's last arrives as zeros for the codes, and multiplies zero
        // activations (a zero-sized buffer, or the LDS form's zero step); the decoded weights of zero codes are finite,
        // so the products add nothing. (Branches here also cost the compiler its count of the loads in flight: it
        // then drains them all at every join.)
        if constexpr (kAhead) {
            GemvStep<CB, WIDE, RB, BT> words[2];
            uint4v xw[2][RB];  // XLds: the activations of the step being decoded and of the next, read beside the words
            stage_step(ring[0], 0u);
            load_step(static_cast<uint32_t>(ST), ring[0]);
            words[0].fetch(stage, BT * kTileSlot, kTileSlot, plan);
            fetch_x(0u, xw[0]);
            uint32_t i = 0;
            do {
#pragma unroll
                for (int s = 0; s < ST; ++s) {
                    const uint32_t step = i + static_cast<uint32_t>(s);
                    const int sn = (s + 1) % ST;  // the ring slot of step + 1
                    __builtin_amdgcn_sched_barrier(0);
                    stage_step(ring[sn], static_cast<uint32_t>(sn & 1));
                    load_step(step + 1u + ST, ring[sn]);
                    words[sn & 1].fetch(stage + static_cast<uint32_t>(sn & 1) * kBuf, BT * kTileSlot, kTileSlot, plan);
                    fetch_x(step + 1u, xw[sn & 1]);
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (kXLds) words[s & 1].consume(plan, wbits, xw[s & 1], acc);
                    else words[s & 1].consume(plan, wbits, xr[s], acc);
                    __builtin_amdgcn_sched_barrier(0);
                    load_x(step + ST, xr[s]);
                }
                i += ST;
            } while (i < steps);
        } else {
            GemvStep<CB, WIDE, RB, BT> words;
            uint4v xw[RB];
            stage_step(ring[0], 0u);
            load_step(static_cast<uint32_t>(ST), ring[0]);
            uint32_t i = 0;
            do {
#pragma unroll
                for (int s = 0; s < ST; ++s) {
                    const uint32_t step = i + static_cast<uint32_t>(s);
                    const int sn = (s + 1) % ST;
                    __builtin_amdgcn_sched_barrier(0);
                    words.fetch(stage, BT * kTileSlot, kTileSlot, plan);
                    fetch_x(step, xw);
                    // the next step's tile rows take the buffer behind these reads (LDS keeps a wave's order)
                    stage_step(ring[sn], 0u);
                    load_step(step + 1u + ST, ring[sn]);
                    __builtin_amdgcn_sched_barrier(0);
                    if constexpr (kXLds) words.consume(plan, wbits, xw, acc);
                    else words.consume(plan, wbits, xr[s], acc);
                    __builtin_amdgcn_sched_barrier(0);
                    load_x(step + ST, xr[s]);
                }
                i += ST;
            } while (i < steps);
        }
    }
};

template <int CB, int WIDE, int RB, int BT, typename XSrc>
struct GemvStreamLds {
#ifndef T3_GEMV_LDS_RING_DEPTH
#define T3_GEMV_LDS_RING_DEPTH 4
#endif
    static constexpr int ST = T3_GEMV_LDS_RING_DEPTH;  // steps' slots in the LDS ring: ST - 1 steps in flight under a decode
    static constexpr int R = gemv_step_rows<CB>();   // tile rows a step
    static constexpr bool kAhead = R == 1;            // as GemvStreamRegs: a second set of words, read a step ahead
    static constexpr uint32_t kSlotBytes = static_cast<uint32_t>(R) * kRowSlot;   // LDS bytes a step
    static constexpr uint32_t kStageBytes = static_cast<uint32_t>(ST) * kSlotBytes;
    static constexpr bool kXLds = __is_same(XSrc, XLds);
    static constexpr int kStepLoads = kXLds ? R : R + RB;      // loads a step
    static constexpr uint32_t kSlot = kRowSlot / BT;           // LDS bytes a tile's slot
    static constexpr uint32_t kLanesATile = 64u / BT;
    static_assert(ST >= 4 && ST % 2 == 0, "word sets alternate by ring slot parity; two steps in flight at least");
    static_assert(BT == 4 || BT == 8, "a tile's slot holds any tile at four tiles a load, up to 128 bytes at eight");

    uint32_t wstep, steps, n, wbits, lane;
    XSrc xs;
    uint32_t xoff[RB];
    unsigned char* stage;
    uint32_t w_lo, w_hi, span_bytes, w_voff, stage_lds;
    uint4v xr[kXLds ? 1 : ST][RB];  // XGlobal: the fragments in flight, by ring slot

    __device__ __forceinline__ GemvStreamLds(const uint32_t* wbase, uint32_t wstep_, uint32_t per_, uint32_t n_,
                                             uint32_t wbits_, const XSrc& xs_, const uint32_t (&xoff_)[RB],
                                             unsigned char* stage_, uint32_t lane_)
        : wstep(wstep_), steps(per_ / static_cast<uint32_t>(R)), n(n_), wbits(wbits_), lane(lane_), xs(xs_), stage(stage_) {
#pragma unroll
        for (int r = 0; r < RB; ++r) xoff[r] = xoff_[r];
        const uint32_t tile_bytes = 2u * n;
        const uint64_t addr = reinterpret_cast<uint64_t>(wbase);
        w_lo = static_cast<uint32_t>(addr);
        w_hi = static_cast<uint32_t>(addr >> 32) & 0xFFFFu;
        // bytes from the wave's first tile row to the end of its last
        span_bytes = (per_ - 1u) * wstep + static_cast<uint32_t>(BT) * tile_bytes;
        // a lane whose piece starts past its tile brings zeros into the slot's tail
        const uint32_t piece = (lane % kLanesATile) * 16u;
        w_voff = piece < tile_bytes ? (lane / kLanesATile) * tile_bytes + piece : kNoBytes;
        stage_lds = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(stage));
    }

    // step `step`'s loads into ring slot `slot` (a constant once the callers' loops are unrolled)
    __device__ __forceinline__ void issue_step(uint32_t step, int slot) {
        const bool live = step < steps;
        const uint4v wd = {w_lo, w_hi, live ? span_bytes : 0u, 0x00020000u};
#pragma unroll
        for (int j = 0; j < R; ++j)
            load_to_lds(wd, stage_lds + static_cast<uint32_t>(slot) * kSlotBytes + static_cast<uint32_t>(j) * kRowSlot, w_voff,
                        (step * R + static_cast<uint32_t>(j)) * wstep);
        if constexpr (!kXLds) {
            const __amdgpu_buffer_rsrc_t xd = make_rsrc(xs.base, live ? xs.bytes : 0u);
#pragma unroll
            for (int r = 0; r < RB; ++r) xr[slot][r] = buf_load_u128(xd, xoff[r], xs.first + step * xs.step);
        }
    }

    __device__ __forceinline__ void issue() {
#pragma unroll
        for (int s = 0; s < ST; ++s) issue_step(static_cast<uint32_t>(s), s);
    }

    __device__ __forceinline__ void run(float4v (&acc)[RB][BT]) {
        // The loads are in flight; everything a lane needs to decode is worked out under their latency.
        const QuadPlan<WIDE> plan = quad_plan<WIDE>(n, lane);
        // a step's activations: the LDS form's out of the wave's prepared block (past the last: the zero step), the
        // others out of the register ring
        auto fetch_x = [&](int slot, uint32_t step, uint4v(&xv)[RB]) {
            if constexpr (kXLds) {
                const uint32_t at = step < steps ? step : steps;
#pragma unroll
                for (int r = 0; r < RB; ++r)
                    xv[r] = *reinterpret_cast<const uint4v*>(xs.base + at * (kXldsRows * 64u) + xoff[r]);
            } else {
#pragma unroll
                for (int r = 0; r < RB; ++r) xv[r] = xr[slot][r];
            }
        };
        // No branch inside the ring: a step past the wave's last arrives as zeros for the codes, and multiplies zero
        // activations (a zero-sized buffer, or the LDS form's zero step); the decoded weights of zero codes are finite,
        // so the products add nothing. (An exit after the last live step was tried: a way out of every unrolled position
        // costs the kernel twice its registers.)
        if constexpr (kAhead) {
            // Step s: steps s + 1 .. s + ST - 1 are in flight. Once s + 1 has landed its words are read while step s
            // decodes, and step s's slot (its words went to registers a step ago, and those reads have returned) takes
            // step s + ST's loads.
            GemvStep<CB, WIDE, RB, BT> words[2];
            uint4v xw[2][RB];
            wait_loads<(ST - 1) * kStepLoads>();  // step 0 has landed
            words[0].fetch(stage, kRowSlot, kSlot, plan);
            fetch_x(0, 0u, xw[0]);
            uint32_t i = 0;
            do {
#pragma unroll
                for (int s = 0; s < ST; ++s) {
                    const uint32_t step = i + static_cast<uint32_t>(s);
                    const int sn = (s + 1) % ST;  // the ring slot of step + 1
                    __builtin_amdgcn_sched_barrier(0);
                    wait_loads<(ST - 2) * kStepLoads>();
                    wait_lds_reads();
                    words[sn & 1].fetch(stage + static_cast<uint32_t>(sn) * kSlotBytes, kRowSlot, kSlot, plan);
                    fetch_x(sn, step + 1u, xw[sn & 1]);
                    issue_step(step + static_cast<uint32_t>(ST), s);
                    __builtin_amdgcn_sched_barrier(0);
                    words[s & 1].consume(plan, wbits, xw[s & 1], acc);
                    __builtin_amdgcn_sched_barrier(0);
                }
                i += static_cast<uint32_t>(ST);
            } while (i < steps);
        } else {
            // Step s: once it has landed (steps s + 1 .. s + ST - 1 in flight) its words are read and decoded, then its
            // slot takes step s + ST's loads.
            GemvStep<CB, WIDE, RB, BT> words;
            uint4v xw[RB];
            uint32_t i = 0;
            do {
#pragma unroll
                for (int s = 0; s < ST; ++s) {
                    const uint32_t step = i + static_cast<uint32_t>(s);
                    __builtin_amdgcn_sched_barrier(0);
                    wait_loads<(ST - 1) * kStepLoads>();
                    words.fetch(stage + static_cast<uint32_t>(s) * kSlotBytes, kRowSlot, kSlot, plan);
                    fetch_x(s, step, xw);
                    __builtin_amdgcn_sched_barrier(0);
                    words.consume(plan, wbits, xw, acc);
                    __builtin_amdgcn_sched_barrier(0);
                    wait_lds_reads();
                    issue_step(step + static_cast<uint32_t>(ST), s);
                }
                i += static_cast<uint32_t>(ST);
            } while (i < steps);
        }
        wait_loads<0>();  // the steps past the last still land (as zeros): the slots' memory is not free before
    }
};

// LDS: the direct-to-LDS ring; else the register ring
// The stream of the measured LDS-table form (t3_dense.hip, dense_gemv_tab): GemvStreamRegs' register ring at two tile
// rows a step, cut down to what fits beside a 128 KB table: the narrow reader, tiles of whole 16-byte pieces and at most
// 128 bytes (up to four bits a weight), packed in the stage (R x BT x 128 bytes a wave), ST steps in flight.
template <int BT, int ST>
struct GemvStreamTab {
    static constexpr int R = 2;
    static constexpr uint32_t kRowBytes = static_cast<uint32_t>(BT) * 128u;
    static constexpr uint32_t kStageBytes = static_cast<uint32_t>(R) * kRowBytes;
    const uint32_t* wbase;
    uint32_t wstep, steps, n, wbits, lane;
    XGlobal xs;
    uint32_t xoff;
    unsigned char* stage;
    uint32_t span_bytes, voff;
    uint4v ring[ST][R];
    uint4v xr[ST][1];

    __device__ __forceinline__ GemvStreamTab(const uint32_t* wbase_, uint32_t wstep_, uint32_t per_, uint32_t n_,
                                             uint32_t wbits_, const XGlobal& xs_, uint32_t xoff_, unsigned char* stage_,
                                             uint32_t lane_)
        : wbase(wbase_), wstep(wstep_), steps(per_ / 2u), n(n_), wbits(wbits_), lane(lane_), xs(xs_), xoff(xoff_),
          stage(stage_) {
        const uint32_t chunk_bytes = static_cast<uint32_t>(BT) * 2u * n;
        span_bytes = (per_ - 1u) * wstep + chunk_bytes;
        voff = lane * 16u < chunk_bytes ? lane * 16u : kNoBytes;
    }
    __device__ __forceinline__ void load_step(uint32_t step, uint4v (&dst)[R]) const {
        const __amdgpu_buffer_rsrc_t res = make_rsrc(wbase, step < steps ? span_bytes : 0u);
#pragma unroll
        for (int j = 0; j < R; ++j) dst[j] = buf_load_u128(res, voff, (step * R + static_cast<uint32_t>(j)) * wstep);
    }
    __device__ __forceinline__ void load_x(uint32_t step, uint4v (&dst)[1]) const {
        const __amdgpu_buffer_rsrc_t res = make_rsrc(xs.base, step < steps ? xs.bytes : 0u);
        dst[0] = buf_load_u128(res, xoff, xs.first + step * xs.step);
    }
    __device__ __forceinline__ void issue() {
#pragma unroll
        for (int s = 0; s < ST; ++s) {
            load_step(static_cast<uint32_t>(s), ring[s]);
            load_x(static_cast<uint32_t>(s), xr[s]);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    __device__ __forceinline__ void run(float4v (&acc)[1][BT]) {
        const uint32_t tile_bytes = 2u * n;
        const QuadPlan<kNarrow> plan = quad_plan<kNarrow>(n, lane);
        const bool writer = lane * 16u < static_cast<uint32_t>(BT) * tile_bytes;
        auto stage_step = [&](const uint4v (&v)[R]) {
            if (writer) {
#pragma unroll
                for (int j = 0; j < R; ++j)
                    *reinterpret_cast<uint4v*>(stage + static_cast<uint32_t>(j) * kRowBytes + lane * 16u) = v[j];
            }
        };
        GemvStep<kMcgTab, kNarrow, 1, BT> words;
        stage_step(ring[0]);
        load_step(static_cast<uint32_t>(ST), ring[0]);
        uint32_t i = 0;
        do {
#pragma unroll
            for (int s = 0; s < ST; ++s) {
                const uint32_t step = i + static_cast<uint32_t>(s);
                const int sn = (s + 1) % ST;
                __builtin_amdgcn_sched_barrier(0);
                words.fetch(stage, kRowBytes, tile_bytes, plan);
                stage_step(ring[sn]);
                load_step(step + 1u + ST, ring[sn]);
                __builtin_amdgcn_sched_barrier(0);
                words.consume(plan, wbits, xr[s], acc);
                __builtin_amdgcn_sched_barrier(0);
                load_x(step + ST, xr[s]);
            }
            i += ST;
        } while (i < steps);
    }
};

template <bool LDS, int CB, int WIDE, int RB, int BT, typename XSrc>
using GemvStream = std::conditional_t<LDS, GemvStreamLds<CB, WIDE, RB, BT, XSrc>, GemvStreamRegs<CB, WIDE, RB, BT, XSrc>>;

}  // namespace t3
