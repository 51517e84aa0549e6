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
constexpr uint32_t kXldsRows = 4u;    // activation rows the in-LDS form of the prepared input holds
constexpr uint32_t kRowSlot = 1024u;  // LDS ring: bytes one load of a wave fills: 64 lanes x 16 bytes
constexpr uint32_t kNoBytes = 0x80000000u;  // a lane offset no buffer reaches: zeros, no traffic

// Where a wave's prepared activations come from.
struct XGlobal {            // doubled f16 in quad order, 64 bytes a (row, input tile)
    const uint32_t* base;
    uint64_t bytes;
    uint32_t first;         // byte offset of the wave's first input tile
    uint32_t step;          // bytes from one input tile to the next: 64 where a row's tiles are adjacent ([rows][in]),
                            // rows x 64 where a tile's rows are ([in / 16][rows][16]: the fragment of one tile row is one
                            // contiguous piece, whole cache lines whatever the rows)
};
struct XLds {               // the wave's own [per + 1][kXldsRows][64 bytes], written by the in-kernel prepare;
    const unsigned char* base;  // the last tile row all zeros: what a row past the wave's last multiplies by
};

// XGlobal: the byte offset, inside one tile row's activations, of a lane's piece of a B fragment: activation row
// lane % 16 of the block lies `row_bytes` into them, the lane's eight K slots are its 16-byte piece lane / 16
// (kNoBytes: that fragment row stays zero).
__device__ __forceinline__ uint32_t x_frag_offset(uint32_t lane, bool live, uint32_t row_bytes) {
    return live ? row_bytes + (lane >> 4) * 16u : kNoBytes;
}

// One wave's stream over `per` tile rows, either form. Construct, `issue()` the first loads, do whatever else the
// kernel has to do while they fly (the one-launch form prepares its activations there), then `run()`.
//
// wbase: the wave's first tile row (tile 0 of its BT); wstep: bytes from one tile row to the next; per: tile rows.
// xoff[r]: XGlobal: x_frag_offset of block r's fragment; XLds: the lane's byte offset of block r's activation row plus
// its quad inside a tile row's kXldsRows x 64 bytes. stage: the wave's own LDS bytes (kStageBytes), 16-byte aligned.
// run(): acc[r][t] += the 16 x 16 product of activation block r and tile t, summed over the wave's tile rows in order;
// when it returns none of the wave's loads is in flight and the stage's memory is free.

template <int CB, int WIDE, int RB, int BT, typename XSrc>
struct GemvStreamRegs {
    static constexpr int ST = 2;  // tile rows in flight in the register ring
    // LDS bytes one wave's stage takes: two buffers of BT tile slots, then a dump where the lanes past a tile row's last
    // byte put their (zero) registers, so the store needs neither a branch nor a per-lane buffer offset: the dump is
    // 512 bytes plus one buffer's length, because a store to buffer 1 adds that length for every lane alike
    static constexpr uint32_t kStageBytes = 3u * BT * kTileSlot + 512u;
    static constexpr bool kXLds = __is_same(XSrc, XLds);
    static_assert(ST % 2 == 0, "stage buffers and word sets alternate by ring slot parity");

    const uint32_t* wbase;
    uint32_t wstep, per, n, wbits, lane;
    XSrc xs;
    uint32_t xoff[RB];
    unsigned char* stage;
    uint32_t span_bytes, voff;
    // Three overlapped pipelines, all in the wave's own program order:
    //   global -> registers   ST tile rows ahead (ring), the activations beside them: the load counter retires in
    //                         order, so a load issued later than a row's would hold that row's wait back to its lead;
    //   registers -> LDS -> registers   one row ahead (two stage buffers, two word sets by row parity);
    //   decode + MFMA         the row whose words are already in registers.
    uint4v ring[ST];
    uint4v xr[ST][RB];

    __device__ __forceinline__ GemvStreamRegs(const uint32_t* wbase_, uint32_t wstep_, uint32_t per_, uint32_t n_,
                                          uint32_t wbits_, const XSrc& xs_, const uint32_t (&xoff_)[RB],
                                          unsigned char* stage_, uint32_t lane_)
        : wbase(wbase_), wstep(wstep_), per(per_), n(n_), wbits(wbits_), lane(lane_), xs(xs_), stage(stage_) {
#pragma unroll
        for (int r = 0; r < RB; ++r) xoff[r] = xoff_[r];
        const uint32_t chunk_bytes = static_cast<uint32_t>(BT) * 2u * n;  // a multiple of 16: BT is 4 or 8, n even
        // bytes from the wave's first tile row to the end of its last (the range check covers the scalar offset too)
        span_bytes = (per - 1u) * wstep + chunk_bytes;
        // a lane past the chunk asks for an offset no buffer reaches: zeros, no traffic
        voff = lane * 16u < chunk_bytes ? lane * 16u : kNoBytes;
    }

    __device__ __forceinline__ uint4v load_chunk(uint32_t row) const {
        const __amdgpu_buffer_rsrc_t res = make_rsrc(wbase, row < per ? span_bytes : 0u);
        return buf_load_u128(res, voff, row * wstep);
    }
    __device__ __forceinline__ void load_x(uint32_t row, uint4v (&dst)[RB]) const {
        if constexpr (!kXLds) {
            const __amdgpu_buffer_rsrc_t res = make_rsrc(xs.base, row < per ? xs.bytes : 0u);
            const uint32_t soff = xs.first + row * xs.step;
#pragma unroll
            for (int r = 0; r < RB; ++r) dst[r] = buf_load_u128(res, xoff[r], soff);
        }
    }

    __device__ __forceinline__ void issue() {
#pragma unroll
        for (int s = 0; s < ST; ++s) {
            ring[s] = load_chunk(static_cast<uint32_t>(s));
            load_x(static_cast<uint32_t>(s), xr[s]);
            __builtin_amdgcn_sched_barrier(0);  // issue order = ring order: the first row's wait must not cover the rest
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
        // into the dump behind both buffers); b / tile_bytes by a 16-bit reciprocal, exact for b < 1024 and
        // tile_bytes >= 32
        const bool writer = lane * 16u < chunk_bytes;
        const uint32_t inv_tile = (1u << 16) / tile_bytes + 1u;
        uint32_t put[4];
#pragma unroll
        for (uint32_t j = 0; j < 4u; ++j) {
            const uint32_t b = lane * 16u + 4u * j;
            const uint32_t t = (b * inv_tile) >> 16;
            put[j] = writer ? t * kTileSlot + (b - t * tile_bytes) : 2u * BT * kTileSlot + (lane & 31u) * 16u + 4u * j;
        }
        // where the lane's quad words sit inside a tile slot
        const uint32_t get_bp = plan.ib_prev * 4u, get_bl = plan.ib_last * 4u;
        const uint32_t get_ap = plan.ia_prev * 4u, get_al = plan.ia_last * 4u;

        auto stage_chunk = [&](const uint4v& v, uint32_t parity) {
            if constexpr (W16) {
                *reinterpret_cast<uint4v*>(stage + parity * (BT * kTileSlot) + put[0]) = v;
            } else {
#pragma unroll
                for (uint32_t j = 0; j < 4u; ++j)
                    *reinterpret_cast<uint32_t*>(stage + parity * (BT * kTileSlot) + put[j]) = v[j];
            }
        };
        // a tile row's words, read back from the stage into registers one row ahead of their decode
        auto fetch = [&](uint32_t parity, uint32_t row, QuadWords<WIDE>(&wd)[BT], uint4v(&xv)[RB]) {
            const unsigned char* buf = stage + parity * (BT * kTileSlot);
#pragma unroll
            for (int t = 0; t < BT; ++t) {
                const unsigned char* slot = buf + static_cast<uint32_t>(t) * kTileSlot;
                wd[t].b_prev = *reinterpret_cast<const uint32_t*>(slot + get_bp);
                wd[t].b_last = *reinterpret_cast<const uint32_t*>(slot + get_bl);
                if constexpr (WIDE == kWide) {
                    wd[t].a_prev = *reinterpret_cast<const uint32_t*>(slot + get_ap);
                    wd[t].a_last = *reinterpret_cast<const uint32_t*>(slot + get_al);
                }
            }
            if constexpr (kXLds) {
                const uint32_t xrow = row < per ? row : per;  // past the last: the zero row
#pragma unroll
                for (int r = 0; r < RB; ++r)
                    xv[r] = *reinterpret_cast<const uint4v*>(xs.base + xrow * (kXldsRows * 64u) + xoff[r]);
            }
        };
        auto consume = [&](const QuadWords<WIDE>(&wd)[BT], const uint4v(&xv)[RB]) {
#pragma unroll
            for (int t = 0; t < BT; ++t) {
                uint32_t cw[4];
                quad_codewords<WIDE>(wd[t], plan, wbits, cw);
                uint4v a;
#pragma unroll
                for (int m = 0; m < 4; ++m) a[m] = weight_pair<CB>(cw[m]);
#pragma unroll
                for (int r = 0; r < RB; ++r)
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        __builtin_bit_cast(half8, a), __builtin_bit_cast(half8, xv[r]), acc[r][t], 0, 0, 0);
            }
        };

        QuadWords<WIDE> words[2][BT];
        uint4v xw[2][RB];  // XLds: the activations of the row being decoded and of the next, read beside the words
        stage_chunk(ring[0], 0u);
        ring[0] = load_chunk(ST);
        fetch(0u, 0u, words[0], xw[0]);
        // No branch inside the ring: a row past the wave's last arrives as zeros for the codes, and multiplies zero
        // activations (a zero-sized buffer, or the LDS form's zero row); the decoded weights of zero codes are finite,
        // so the products add nothing. (Branches here also cost the compiler its count of the loads in flight: it
        // then drains them all at every join.)
        uint32_t i = 0;
        do {
#pragma unroll
            for (int s = 0; s < ST; ++s) {
                const uint32_t row = i + static_cast<uint32_t>(s);
                const int sn = (s + 1) % ST;  // the ring slot of row + 1
                __builtin_amdgcn_sched_barrier(0);
                stage_chunk(ring[sn], static_cast<uint32_t>(sn & 1));
                ring[sn] = load_chunk(row + 1u + ST);
                fetch(static_cast<uint32_t>(sn & 1), row + 1u, words[sn & 1], xw[sn & 1]);
                __builtin_amdgcn_sched_barrier(0);
                if constexpr (kXLds) consume(words[s & 1], xw[s & 1]);
                else consume(words[s & 1], xr[s]);
                __builtin_amdgcn_sched_barrier(0);
                load_x(row + ST, xr[s]);
            }
            i += ST;
        } while (i < per);
    }
};


template <int CB, int WIDE, int RB, int BT, typename XSrc>
struct GemvStreamLds {
    static constexpr int ST = 4;  // tile rows' slots in the LDS ring: ST - 1 rows in flight under a decode
    static constexpr uint32_t kStageBytes = static_cast<uint32_t>(ST) * kRowSlot;
    static constexpr bool kXLds = __is_same(XSrc, XLds);
    static constexpr int kRowLoads = kXLds ? 1 : 1 + RB;       // loads a tile row
    static constexpr uint32_t kSlot = kRowSlot / BT;           // LDS bytes a tile's slot
    static constexpr uint32_t kLanesATile = 64u / BT;
    static_assert(ST >= 4 && ST % 2 == 0, "word sets alternate by ring slot parity; two rows in flight at least");
    static_assert(BT == 4 || BT == 8, "a tile's slot holds any tile at four tiles a load, up to 128 bytes at eight");

    uint32_t wstep, per, n, wbits, lane;
    XSrc xs;
    uint32_t xoff[RB];
    unsigned char* stage;
    uint32_t w_lo, w_hi, span_bytes, w_voff, stage_lds;
    uint4v xr[kXLds ? 1 : ST][RB];  // XGlobal: the fragments in flight, by ring slot

    __device__ __forceinline__ GemvStreamLds(const uint32_t* wbase, uint32_t wstep_, uint32_t per_, uint32_t n_,
                                          uint32_t wbits_, const XSrc& xs_, const uint32_t (&xoff_)[RB],
                                          unsigned char* stage_, uint32_t lane_)
        : wstep(wstep_), per(per_), n(n_), wbits(wbits_), lane(lane_), xs(xs_), stage(stage_) {
#pragma unroll
        for (int r = 0; r < RB; ++r) xoff[r] = xoff_[r];
        const uint32_t tile_bytes = 2u * n;
        const uint64_t addr = reinterpret_cast<uint64_t>(wbase);
        w_lo = static_cast<uint32_t>(addr);
        w_hi = static_cast<uint32_t>(addr >> 32) & 0xFFFFu;
        // bytes from the wave's first tile row to the end of its last
        span_bytes = (per - 1u) * wstep + static_cast<uint32_t>(BT) * tile_bytes;
        // a lane whose piece starts past its tile brings zeros into the slot's tail
        const uint32_t piece = (lane % kLanesATile) * 16u;
        w_voff = piece < tile_bytes ? (lane / kLanesATile) * tile_bytes + piece : kNoBytes;
        stage_lds = static_cast<uint32_t>(reinterpret_cast<uintptr_t>(stage));
    }

    // tile row `row`'s loads into ring slot `slot` (a constant once the callers' loops are unrolled)
    __device__ __forceinline__ void issue_row(uint32_t row, int slot) {
        const bool live = row < per;
        load_to_lds(uint4v{w_lo, w_hi, live ? span_bytes : 0u, 0x00020000u},
                    stage_lds + static_cast<uint32_t>(slot) * kRowSlot, w_voff, row * wstep);
        if constexpr (!kXLds) {
            const __amdgpu_buffer_rsrc_t xd = make_rsrc(xs.base, live ? xs.bytes : 0u);
#pragma unroll
            for (int r = 0; r < RB; ++r) xr[slot][r] = buf_load_u128(xd, xoff[r], xs.first + row * xs.step);
        }
    }

    __device__ __forceinline__ void issue() {
#pragma unroll
        for (int s = 0; s < ST; ++s) issue_row(static_cast<uint32_t>(s), s);
    }

    __device__ __forceinline__ void run(float4v (&acc)[RB][BT]) {
        // The loads are in flight; everything a lane needs to decode is worked out under their latency.
        const QuadPlan<WIDE> plan = quad_plan<WIDE>(n, lane);
        // where the lane's quad words sit inside a tile's slot
        const uint32_t get_bp = plan.ib_prev * 4u, get_bl = plan.ib_last * 4u;
        const uint32_t get_ap = plan.ia_prev * 4u, get_al = plan.ia_last * 4u;

        // a tile row's words, read back from its slot into registers one row ahead of their decode
        auto fetch = [&](int slot, uint32_t row, QuadWords<WIDE>(&wd)[BT], uint4v(&xv)[RB]) {
            const unsigned char* buf = stage + static_cast<uint32_t>(slot) * kRowSlot;
#pragma unroll
            for (int t = 0; t < BT; ++t) {
                const unsigned char* tile = buf + static_cast<uint32_t>(t) * kSlot;
                wd[t].b_prev = *reinterpret_cast<const uint32_t*>(tile + get_bp);
                wd[t].b_last = *reinterpret_cast<const uint32_t*>(tile + get_bl);
                if constexpr (WIDE == kWide) {
                    wd[t].a_prev = *reinterpret_cast<const uint32_t*>(tile + get_ap);
                    wd[t].a_last = *reinterpret_cast<const uint32_t*>(tile + get_al);
                }
            }
            if constexpr (kXLds) {
                const uint32_t xrow = row < per ? row : per;  // past the last: the zero row
#pragma unroll
                for (int r = 0; r < RB; ++r)
                    xv[r] = *reinterpret_cast<const uint4v*>(xs.base + xrow * (kXldsRows * 64u) + xoff[r]);
            } else {
#pragma unroll
                for (int r = 0; r < RB; ++r) xv[r] = xr[slot][r];
            }
        };
        auto consume = [&](const QuadWords<WIDE>(&wd)[BT], const uint4v(&xv)[RB]) {
#pragma unroll
            for (int t = 0; t < BT; ++t) {
                uint32_t cw[4];
                quad_codewords<WIDE>(wd[t], plan, wbits, cw);
                uint4v a;
#pragma unroll
                for (int m = 0; m < 4; ++m) a[m] = weight_pair<CB>(cw[m]);
#pragma unroll
                for (int r = 0; r < RB; ++r)
                    acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        __builtin_bit_cast(half8, a), __builtin_bit_cast(half8, xv[r]), acc[r][t], 0, 0, 0);
            }
        };

        QuadWords<WIDE> words[2][BT];
        uint4v xw[2][RB];
        wait_loads<(ST - 1) * kRowLoads>();  // row 0 has landed
        fetch(0, 0u, words[0], xw[0]);
        // No branch inside the ring: a row past the wave's last arrives as zeros for the codes, and multiplies zero
        // activations (a zero-sized buffer, or the LDS form's zero row); the decoded weights of zero codes are finite,
        // so the products add nothing. (An exit after the last live row was tried: a way out of every unrolled position
        // costs the kernel twice its registers.) The host's partitions give a wave a multiple of the ring's rows.
        // Row r: rows r + 1 .. r + ST - 1 are in flight. Once r + 1 has landed, row r's slot (its words went to
        // registers a row ago, and those reads have returned) takes row r + ST's loads; row r + 1's words are read
        // while row r decodes.
        uint32_t i = 0;
        do {
#pragma unroll
            for (int s = 0; s < ST; ++s) {
                const uint32_t row = i + static_cast<uint32_t>(s);
                const int sn = (s + 1) % ST;  // the ring slot of row + 1
                __builtin_amdgcn_sched_barrier(0);
                wait_loads<(ST - 2) * kRowLoads>();
                wait_lds_reads();
                fetch(sn, row + 1u, words[sn & 1], xw[sn & 1]);
                issue_row(row + static_cast<uint32_t>(ST), s);
                __builtin_amdgcn_sched_barrier(0);
                consume(words[s & 1], xw[s & 1]);
                __builtin_amdgcn_sched_barrier(0);
            }
            i += static_cast<uint32_t>(ST);
        } while (i < per);
        wait_loads<0>();  // the rows past the last still land (as zeros): the slots' memory is not free before
    }
};


// LDS: the direct-to-LDS ring; else the register ring
template <bool LDS, int CB, int WIDE, int RB, int BT, typename XSrc>
using GemvStream = std::conditional_t<LDS, GemvStreamLds<CB, WIDE, RB, BT, XSrc>, GemvStreamRegs<CB, WIDE, RB, BT, XSrc>>;

}  // namespace t3
