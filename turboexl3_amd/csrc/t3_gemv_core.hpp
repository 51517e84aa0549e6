// The streaming core every decode-row GEMV of this library runs: one wave walks `per` tile rows of a trellis matrix
// (BT adjacent 16x16 tiles a row), decodes each tile a quad of weights a lane straight into the A fragment of
// v_mfma_f32_16x16x32_f16, and multiplies by up to 32 prepared activation rows held as B fragments.
//
// Memory path. A tile row's BT tiles are contiguous (BT * 2n bytes <= 1 KB), so the wave fetches them with ONE
// 128-bit buffer load, 16 consecutive bytes a lane: the texture unit sees a fully coalesced stream (a gather of each
// lane's own words costs it many times the cycles, measured). The loaded registers go to a wave-private LDS stage,
// one 256-byte slot a tile, and every lane reads back the two (or four) words its quad needs. ST such loads stay in
// flight in a register ring, fully unrolled, with scalar row offsets: the loop spends no vector ALU on addresses.
// A row past the wave's last is read through a zero-sized buffer: the hardware returns zeros without touching memory.
// LDS operations of one wave complete in order, so the stage needs no barrier.
//
// Sums: each MFMA output element depends on its own activation row alone, and a wave's tile rows are taken in
// ascending order, so a row's partial sum is a function of (matrix, K part, row) only.
#pragma once

#include "t3_decode.hpp"

namespace t3 {

constexpr uint32_t kTileSlot = 256u;  // LDS bytes a staged tile (2n <= 256)

// LDS bytes one wave's stage takes: two buffers of BT tile slots
template <int BT>
constexpr uint32_t gemv_stage_bytes() {
    return 2u * BT * kTileSlot;
}

// wbase: the wave's first tile row (tile 0 of its BT); wstep: bytes from one tile row to the next; per: tile rows.
// xbase/xbytes: the prepared rows (u32 [rows][in], doubled f16 in quad order); xoff[r]: the lane's byte offset of
// block r's activation row plus its quad; xo: byte offset of the wave's first input tile inside a row (tile 64 B).
// stage: the wave's own LDS bytes (gemv_stage_bytes<BT>()), 16-byte aligned.
// acc[r][t] += the 16 x 16 product of activation block r and tile t, summed over the wave's tile rows in order.
template <int CB, bool WIDE, int RB, int BT, int ST>
__device__ __forceinline__ void gemv_stream(const uint32_t* wbase, uint32_t wstep, uint32_t per, uint32_t n,
                                            const QuadPlan<WIDE>& plan, uint32_t wbits, const uint32_t* xbase,
                                            uint64_t xbytes, const uint32_t (&xoff)[RB], uint32_t xo,
                                            unsigned char* stage, uint32_t lane, float4v (&acc)[RB][BT]) {
    const uint32_t tile_bytes = 2u * n;
    const uint32_t chunk_bytes = static_cast<uint32_t>(BT) * tile_bytes;  // a multiple of 16: BT is 4 or 8, n even
    // bytes from the wave's first tile row to the end of its last (the range check covers the scalar offset too)
    const uint32_t span_bytes = (per - 1u) * wstep + chunk_bytes;
    // a lane past the chunk asks for an offset no buffer reaches: zeros, no traffic
    const uint32_t voff = lane * 16u < chunk_bytes ? lane * 16u : 0x40000000u;
    // where the lane's four loaded dwords land: tile slot + offset inside the tile
    uint32_t put[4];
#pragma unroll
    for (uint32_t j = 0; j < 4u; ++j) {
        const uint32_t b = lane * 16u + 4u * j;
        const uint32_t t = b / tile_bytes;
        put[j] = t * kTileSlot + (b - t * tile_bytes);
    }
    const bool writer = lane * 16u < chunk_bytes;
    // where the lane's quad words sit inside a tile slot
    const uint32_t get_bp = plan.ib_prev * 4u, get_bl = plan.ib_last * 4u;
    const uint32_t get_ap = plan.ia_prev * 4u, get_al = plan.ia_last * 4u;

    auto load_chunk = [&](uint32_t row) -> uint4v {
        const __amdgpu_buffer_rsrc_t res = make_rsrc(wbase, row < per ? span_bytes : 0u);
        return buf_load_u128(res, voff, row * wstep);
    };
    auto load_x = [&](uint32_t row, uint4v(&dst)[RB]) {
        const __amdgpu_buffer_rsrc_t res = make_rsrc(xbase, row < per ? xbytes : 0u);
        const uint32_t soff = xo + row * 64u;
#pragma unroll
        for (int r = 0; r < RB; ++r) dst[r] = buf_load_u128(res, xoff[r], soff);
    };
    auto stage_chunk = [&](const uint4v& v, unsigned char* buf) {
        if (writer) {
#pragma unroll
            for (uint32_t j = 0; j < 4u; ++j) *reinterpret_cast<uint32_t*>(buf + put[j]) = v[j];
        }
    };
    auto consume = [&](const unsigned char* buf, const uint4v(&xv)[RB]) {
#pragma unroll
        for (int t = 0; t < BT; ++t) {
            const unsigned char* slot = buf + static_cast<uint32_t>(t) * kTileSlot;
            QuadWords<WIDE> words;
            words.b_prev = *reinterpret_cast<const uint32_t*>(slot + get_bp);
            words.b_last = *reinterpret_cast<const uint32_t*>(slot + get_bl);
            if constexpr (WIDE) {
                words.a_prev = *reinterpret_cast<const uint32_t*>(slot + get_ap);
                words.a_last = *reinterpret_cast<const uint32_t*>(slot + get_al);
            }
            uint32_t cw[4];
            quad_codewords<WIDE>(words, plan, wbits, cw);
            uint4v a;
#pragma unroll
            for (int m = 0; m < 4; ++m) a[m] = weight_pair<CB>(cw[m]);
#pragma unroll
            for (int r = 0; r < RB; ++r)
                acc[r][t] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(half8, a),
                                                                   __builtin_bit_cast(half8, xv[r]), acc[r][t], 0, 0, 0);
        }
    };

    // The activations ride the same ring as the codes: the load counter retires in order, so an activation load
    // issued later than a tile row's would hold that row's wait back to the activations' shorter lead.
    static_assert(ST % 2 == 0, "the LDS stage alternates two buffers by ring slot parity");
    uint4v ring[ST];
    uint4v xr[ST][RB];
#pragma unroll
    for (int s = 0; s < ST; ++s) {
        load_x(static_cast<uint32_t>(s), xr[s]);
        ring[s] = load_chunk(static_cast<uint32_t>(s));
        __builtin_amdgcn_sched_barrier(0);  // issue order = ring order: the first row's wait must not cover the rest
    }
    for (uint32_t i = 0; i < per; i += ST) {
#pragma unroll
        for (int s = 0; s < ST; ++s) {
            const uint32_t row = i + static_cast<uint32_t>(s);
            unsigned char* buf = stage + static_cast<uint32_t>(s & 1) * (BT * kTileSlot);
            __builtin_amdgcn_sched_barrier(0);
            if (row < per) {
                stage_chunk(ring[s], buf);
                uint4v xv[RB];
#pragma unroll
                for (int r = 0; r < RB; ++r) xv[r] = xr[s][r];
                __builtin_amdgcn_sched_barrier(0);
                ring[s] = load_chunk(row + ST);
                load_x(row + ST, xr[s]);
                __builtin_amdgcn_sched_barrier(0);
                consume(buf, xv);
            }
        }
    }
}

}  // namespace t3
