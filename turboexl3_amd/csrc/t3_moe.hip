// Routed experts at decode rows on gfx950: the split-K GEMV chain over gathered top-k experts, no decoded weight
// written anywhere (turboexl3 src/core/decode.zig:274-517 form 3 / form 9; roles of src/hip/plan.zig:294-364).
//
// Per routed pair ("row-slot") rk = row * KT + k, expert e (profile "exl3": format.project's rounding points, the
// reference's src/core/ref.zig:154-190):
//   prepare   xg, xu = f16(H128(f16(x) * suh_e) / sqrt(128)) with the gate's and the up's own suh;
//   gate|up   zg, zu = xg * Wg_e, xu * Wu_e, split over K parts, planes summed in part order;
//   mid       g, u = finish(zg), finish(zu) -> clamp (gate from above, up both ways) -> h = f16(silu(g) * u)
//             -> the down's prepare of h with down_suh_e;
//   down      zd = hd * Wd_e;
//   combine   per row: acc = fma(score_k, finish(zd_k), acc) in slot order, then y's dtype.
// A shared expert rides the same launches as slots K..KT-1 of every row, read from its own bank at weight 1.
// One wave serves one row-slot's K part with the dense path's streaming core; the matrix core runs one live row of 16.
// Launch forms: five launches (prepare apart), four (each gate|up wave prepares its own 128-block in LDS), two (the mid
// stage and the combine run by the last workgroup to arrive at a block, or the mid stage by the down launch's own waves),
// or six (the five behind a grouping launch: the row-slots that read one expert served together). The same statements in
// the same order a row-slot, so the same bytes.

#include "t3_gemv_core.hpp"
#include "t3_kernels.hpp"
#include "t3_routed.hpp"
#include "t3_stages.hpp"

namespace t3 {
namespace {

// Grid (hidden / 128, RKT), 64 threads: the five-launch form's prepare.
template <int PROF>
__global__ void __launch_bounds__(64) moe_prep(const MoeLaunch a) {
    routed_prep_block<false, PROF>(a, blockIdx.y, blockIdx.y, blockIdx.x, threadIdx.x);
}

// Grid (out / 16 / BT, RKT * NPROJ, KS), 256 threads. NPROJ 2: gate (proj 0) and up (proj 1), hidden -> inter;
// NPROJ 1: down, inter -> hidden. Wave sg of slice blockIdx.z takes K part 4 z + sg of `parts` (a part: `per` input
// tiles). z[proj]: f32 [KS][RKT][out], the four waves' sums, wave 0 first. XLDS (gate|up only, per == 8): the wave
// prepares its own 128-block of x in LDS.
//
// XLDS on the down launch (per == 8: a wave's eight input tiles are one 128-block): the wave makes its input itself,
// running the mid stage of that block over the gate|up launch's planes: the stage no longer waits for a hand-off inside
// a launch but is run by all sixteen column workgroups of a slot. Measured against the arriving gate|up launch with
// eight tiles a down wave (us a call): 3 rows 35.0 against 35.5, 4 rows 38.0 against 38.6, 8 rows 57.9 against 56.0,
// 16 rows 98.6 against 94.7: served up to kMidInDownRows = 4 rows. (With four tiles a down wave, an earlier form, it won
// up to two rows only: one row 25.3 against 26.5, two 29.7 against 31.2, three 38.0 against 37.3.) A workgroup of eight
// waves over the same 128 columns (four tiles a load a wave, two column groups: the arrivals a counter unchanged, the
// waves half as long) was measured for this launch as well: one row 15.3 -> 15.0 us, two 16.4 -> 17.5, three 18.3 ->
// 21.4: every wave of a slot repeats the mid stage, and eight of them do it where four did. Taken out.
//
// ARRIVE: the launch also runs the stage after it. The planes are stored device-coherently, every workgroup counts
// itself in at its 128-column block, and the last to arrive runs that block's next stage on the complete planes:
// gate|up -> the slot's mid block (counter a (row-slot, block of inter)); down -> the row's combine block (counter a
// (row, block of hidden); skipped slots count themselves in too). The statements are the chain's, so are the bytes.
constexpr uint32_t kMidInDownRows = kMoeFewRows;

// the register ring: a row-slot's waves walk eight tile rows (the LDS ring pays from about 32 a wave)
constexpr bool kMoeLdsRing = T3_GEMV_LDS_RING_FROM <= 8;

// a wave's share of its workgroup's LDS: its ring while it streams, its partial sums afterwards (the last arriver's
// sixteen finished slots, 8 KB, lie over the first waves' shares)
template <int BT>
constexpr uint32_t role_wave_lds_bytes() {
    constexpr uint32_t stage = GemvStream<kMoeLdsRing, kMcg, kNarrow, 1, BT, XLds>::kStageBytes, red = BT * 4u * 16u;
    return stage > red ? stage : red;
}

// NW: the waves a workgroup, four a K slice. Eight: the workgroup holds both K slices of a down projection that has two
// (an intermediate size of 513 to 1024), one wave a 128-block of the input (a wave past the last block adds zeros), and
// adds their sums as the stage behind the planes would: slice 0's four first, then slice 1's. (Five to eight waves by
// the blocks, their LDS sized by the launch, was measured too: 0.2 to 0.8 us slower at one to three rows than eight
// waves always, and its 320-thread workgroups of 512 experts of 2560 x 640 at four rows no longer fit one round: 30.8
// -> 37.6 us.) smem: the waves' shares; xbase: the waves' prepared activations where the launch makes them (XLDS).
template <int CB, int WIDE, int BT, int NPROJ, bool XLDS, bool ARRIVE, int PROF, int NW>
__device__ __forceinline__ void gemv_role(const MoeLaunch& a, uint32_t blk, uint32_t yidx, uint32_t ksl,
                                          unsigned char* smem, unsigned char* xbase, uint32_t& last_flag, uint32_t* cinfo,
                                          float* cscore) {
    typedef GemvStream<kMoeLdsRing, CB, WIDE, 1, BT, XLds> StreamL;
    typedef GemvStream<kMoeLdsRing, CB, WIDE, 1, BT, XGlobal> StreamG;
    constexpr uint32_t kStage = StreamG::kStageBytes;
    static_assert(kStage <= role_wave_lds_bytes<BT>() && StreamL::kStageBytes <= role_wave_lds_bytes<BT>(), "a wave's ring fits its share");
    constexpr int R = gemv_step_rows<CB>();   // tile rows a step
    // the codebook form says whether MUL1's map is deferred (a.defer repeats it): the other forms' kernels carry none of
    // the map's loads, sums and stores
    constexpr int kDefer = CB == kMul1Defer ? 1 : 0;
    float4v(*red)[BT * 4] = reinterpret_cast<float4v(*)[BT * 4]>(smem);  // the one live row: four lanes a tile a wave
    const uint32_t rk = yidx / NPROJ, proj = yidx % NPROJ;
    const uint32_t sg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63u;
    const SlotRef s = resolve_slot(a, rk);
    // uniform over the workgroup; the down launch's arriving form still has to count a skipped slot in
    if (!s.live && !(ARRIVE && NPROJ == 1)) return;
    if constexpr (ARRIVE && NPROJ == 1) {
        // What the combine will need of the row's slots, fetched now: the workgroup that arrives last would otherwise
        // wait for two dependent loads a slot at the very end of the call. cinfo: the expert, bit 31 for a shared
        // slot, all ones for a skipped one.
        const uint32_t kt = a.topk + a.shared_slots;
        if (threadIdx.x < kt) {
            const SlotRef sk = resolve_slot(a, s.row * kt + threadIdx.x);
            cinfo[threadIdx.x] = !sk.live ? 0xFFFFFFFFu : (sk.shared ? 0x80000000u | sk.e : sk.e);
            // GLM's profile has no scores: every slot's output is stored by itself
            if constexpr (PROF == 0) cscore[threadIdx.x] = sk.shared ? 1.0f : (sk.live ? score_of(a, s.row, threadIdx.x) : 0.0f);
        }
    }
    const RoutedBank& bank = s.shared ? a.shared : a.bank;
    const uint32_t in = NPROJ == 2 ? a.hidden : a.inter, out = NPROJ == 2 ? a.inter : a.hidden;
    const uint32_t n = NPROJ == 2 ? a.n_gu : a.n_dn;
    const uint32_t per = NPROJ == 2 ? a.per_gu : a.per_dn, parts = NPROJ == 2 ? a.parts_gu : a.parts_dn;
    const uint32_t in_tiles = in >> 4, out_tiles = out >> 4, nw = n >> 1;
    const uint32_t* wmat = (NPROJ == 1 ? bank.down_t : (proj ? bank.up_t : bank.gate_t)) +
                           static_cast<size_t>(s.e) * in_tiles * out_tiles * nw;
    const uint32_t part = ksl * NW + sg;
    const uint32_t tk0 = part * per;
    const uint64_t wstride = static_cast<uint64_t>(out_tiles) * nw;
    const uint32_t* wbase = wmat + static_cast<uint64_t>(blk) * BT * nw + tk0 * wstride;
    const uint32_t wstep = static_cast<uint32_t>(wstride) * 4u;
    const uint32_t rkt = a.rows * (a.topk + a.shared_slots);

    float4v acc[1][BT];
#pragma unroll
    for (int t = 0; t < BT; ++t) acc[0][t] = float4v{0.f, 0.f, 0.f, 0.f};

    // The down launch's workgroup holds a slot's complete sums of its 128 columns where it is the only one to make them
    // (one K slice, eight tiles a load): it then finishes them itself (the map, H128, svh: the slot's own statements on
    // the same values) and stores the finished values where the plane would go, and the row's last arriver only adds
    // the slots up in their order. Left to the last arriver, the slots' finishes and their scale loads (an expert's
    // svh comes from HBM) stood one behind the other at the very end of the call: 512 experts of 2048 x 512, one token,
    // the combine 4 us of the down launch's 14.9.
    constexpr bool kMayFinishHere = NPROJ == 1 && ARRIVE && PROF == 0 && BT == 8;
    const bool finish_here = kMayFinishHere && a.ks_dn == 1u;
    float wave_sum = 0.0f;  // the deferred map's block sum of the wave's own 128-block (the mid stage run here)
    float sv_here[2] = {0.0f, 0.0f};
    if constexpr (kMayFinishHere) {
        if (finish_here && sg == 0u && s.live) {  // the scales go out now and are back long before they are needed
            const uint16_t* svh = bank.down_svh + static_cast<size_t>(s.e) * a.hidden + blk * 128u;
            sv_here[0] = half_value(svh[lane]);
            sv_here[1] = half_value(svh[lane + 64u]);
        }
    }

    if (part < parts && s.live) {  // uniform over the wave; a wave past the last part adds zeros below
        uint32_t xoff[1];
        if constexpr (XLDS && NPROJ == 1) {
            // The down's input made here: the wave runs the mid stage of its own 128-block (its eight input tiles) over
            // the gate|up launch's planes and keeps the prepared block in LDS.
            const uint32_t steps = per / R;
            unsigned char* xst = xbase + sg * ((steps + 1u) * (kXldsRows * 64u));
            xoff[0] = (lane >> 4) * 16u;
            StreamL stream(wbase, wstep, per, n, a.wbits, XLds{xst}, xoff, smem + sg * kStage, lane);
            stream.issue();
            uint32_t hh[2];
            float sum;
            routed_mid_values<false, false, PROF, kDefer>(a, s, rk, tk0 >> 3, lane, hh, sum);
            wave_sum = sum;
            // element i = 64 j + lane of the block belongs to step i / (16 R) of the wave's walk
#pragma unroll
            for (uint32_t j = 0; j < 2u; ++j) {
                const uint32_t i = 64u * j + lane;
                x_step_store<R>(xst + ((i / (16u * R)) * kXldsRows) * 64u, i % (16u * R), hh[j]);
            }
            // The row's combine, later in this launch, reads the sum: out of the 128-column block's own copy of hs,
            // [hidden / 128][row-slots][a slot's sums in cache lines of their own], stored by that block's first
            // workgroup column alone. (One copy
            // shared by every column workgroup of the slot takes hundreds of device-coherent stores to the same few
            // cache lines, which serialise: 512 experts of 2560 x 640 at one token, the deferred map, this launch
            // 30.5 us at K3 and 49.6 at K5 against 16.9 and 19.6 for the codebook without the map.)
            if (kDefer && !finish_here && lane == 0u && blk % (8u / BT) == 0u)
                store_coherent(a.hs + (static_cast<size_t>(blk / (8u / BT)) * rkt + rk) * hs_copy_stride(a.inter) + (tk0 >> 3), sum);
            for (uint32_t i = lane; i < kXldsRows * 16u; i += 64u)
                *reinterpret_cast<uint32_t*>(xst + steps * (kXldsRows * 64u) + i * 4u) = 0u;
            stream.run(acc);
        } else if constexpr (XLDS) {
            const uint32_t steps = per / R;
            unsigned char* xst = xbase + sg * ((steps + 1u) * (kXldsRows * 64u));
            xoff[0] = (lane >> 4) * 16u;  // every activation row of the fragment is the slot's one row
            StreamL stream(wbase, wstep, per, n, a.wbits, XLds{xst}, xoff, smem + sg * kStage, lane);
            stream.issue();
            const uint16_t* suh = (proj ? bank.up_suh : bank.gate_suh) + static_cast<size_t>(s.e) * a.hidden;
            const uint32_t blocks = per >> 3;
            for (uint32_t b = 0; b < blocks; ++b) {
                uint32_t hv[2];
                float sum;
                prep_values(a.dtype, a.x, suh, a.hidden, s.row, (tk0 >> 3) + b, lane, hv, sum, PROF == 0);
#pragma unroll
                for (uint32_t j = 0; j < 2u; ++j) {
                    const uint32_t i = b * 128u + lane + 64u * j;  // element of the wave's K part
                    x_step_store<R>(xst + ((i / (16u * R)) * kXldsRows) * 64u, i % (16u * R), hv[j]);
                }
                // every column workgroup of the slot stores the same sum: a handful of plain stores, read by the
                // next launch
                if (kDefer && lane == 0u) {
                    float* at = (proj ? a.su : a.sg) + static_cast<size_t>(rk) * (a.hidden / 128u) + (tk0 >> 3) + b;
                    if constexpr (ARRIVE) store_coherent(at, sum);
                    else *at = sum;
                }
            }
            for (uint32_t i = lane; i < kXldsRows * 16u; i += 64u)
                *reinterpret_cast<uint32_t*>(xst + steps * (kXldsRows * 64u) + i * 4u) = 0u;
            stream.run(acc);
            // (Touching the slot's down trellis from here, so that the down launch behind this one finds it in the
            // memory-side cache, was measured: a piece a wave, the loads left to land by themselves. This launch 8.2 ->
            // 8.9 us at one token, the down launch no shorter, the call 23.65 -> 23.97 us. Taken out.)
        } else {
            const uint32_t* xq = NPROJ == 1 ? a.hd : (proj ? a.xu : a.xg);
            // a row-slot's prepared inputs: 4 bytes an input (doubled f16) at one tile row a step, 2 (plain f16) at two:
            // 64 bytes a step either way. The fragment's row 0 is the slot's row; the other fifteen stay zero.
            constexpr uint32_t kIn = R == 1 ? 4u : 2u;
            xoff[0] = x_frag_offset(lane, (lane & 15u) == 0u, rk * in * kIn);
            StreamG stream(wbase, wstep, per, n, a.wbits,
                           XGlobal{xq, static_cast<uint64_t>(rkt) * in * kIn, (tk0 / R) * 64u, 64u}, xoff, smem + sg * kStage,
                           lane);
            stream.issue();
            stream.run(acc);
        }
    }
    __syncthreads();
    // activation row 0 of the fragment is the slot's row: lanes with lane % 16 == 0 hold its sums
    if ((lane & 15u) == 0u)
#pragma unroll
        for (int t = 0; t < BT; ++t) red[sg][t * 4 + (lane >> 4)] = acc[0][t];
    __syncthreads();
    float* z = NPROJ == 1 ? a.zd : (proj ? a.zu : a.zg);
    float* here = reinterpret_cast<float*>(smem + 4096u);  // finish_here: the 128 sums, then the waves' block sums
    if (threadIdx.x < static_cast<uint32_t>(BT * 4)) {
        const uint32_t i = threadIdx.x, t = i >> 2;
        float4v v = ((red[0][i] + red[1][i]) + red[2][i]) + red[3][i];
        if constexpr (NW == 8) v = v + (((red[4][i] + red[5][i]) + red[6][i]) + red[7][i]);  // plane 0 + plane 1
        float* dst = z + (static_cast<size_t>(ksl) * rkt + rk) * out + (blk * BT + t) * 16u + 4u * (i & 3u);
        if (finish_here) {
            *reinterpret_cast<float4v*>(here + t * 16u + 4u * (i & 3u)) = v;
        } else if constexpr (ARRIVE) {
            if (s.live) store_coherent4(dst, v);
        } else {
            *reinterpret_cast<float4v*>(dst) = v;
        }
    }
    if constexpr (kMayFinishHere) {
        if (finish_here) {
            if constexpr (XLDS) {
                if (lane == 0u) here[128u + sg] = wave_sum;
            }
            __syncthreads();
            if (sg == 0u && s.live) {
                float v[2] = {here[lane], here[lane + 64u]};
                if constexpr (kDefer != 0) {
                    const uint32_t nbi = a.inter / 128u;  // = the waves that hold a block (one K slice)
                    float xsum = 0.0f;
                    if constexpr (XLDS) {
                        for (uint32_t q = 0; q < nbi; ++q) xsum += here[128u + q];  // lane_ordered_sum's order
                    } else {
                        xsum = lane_ordered_sum<false>(a.hs + static_cast<size_t>(rk) * nbi, nbi, lane);
                    }
#pragma unroll
                    for (uint32_t j = 0; j < 2u; ++j) v[j] = __builtin_fmaf(v[j], mul1_a(), mul1_b() * xsum);
                }
                finish_core(v, sv_here, lane);
                float* dst = a.zd + static_cast<size_t>(rk) * a.hidden + blk * 128u;
                store_coherent(dst + lane, v[0]);
                store_coherent(dst + lane + 64u, v[1]);
            }
        }
    }

    if constexpr (ARRIVE) {
        constexpr uint32_t kShare = 8u / BT;  // workgroup columns a 128-column block
        // the last arriver finishes the row's slots sixteen at a time, slot k0 + NW r + wave the wave's r-th
        constexpr uint32_t kMine = 16u / NW;
        const uint32_t b128 = blk / kShare, kt = a.topk + a.shared_slots;
        const uint32_t ks = NPROJ == 2 ? a.ks_gu : a.ks_dn;
        const uint32_t counter = NPROJ == 2 ? arrive_slot(rk * (a.inter / 128u) + b128, rkt * (a.inter / 128u))
                                            : arrive_slot(s.row * (a.hidden / 128u) + b128, a.rows * (a.hidden / 128u));
        const uint32_t full = NPROJ == 2 ? 2u * ks * kShare : kt * ks * kShare;
        wait_stores();
        __syncthreads();
        if (threadIdx.x == 0u) {
            const uint32_t before =
                __hip_atomic_fetch_add(a.arrive + counter, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            last_flag = before == full - 1u;
        }
        __syncthreads();
        if (!last_flag) return;
        if (threadIdx.x == 0u)  // zero again for the next call
            __hip_atomic_store(a.arrive + counter, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if constexpr (NPROJ == 2) {
            if (sg == 0u) routed_mid_block<false, true, PROF, kDefer>(a, s, rk, b128, lane);
        } else if constexpr (PROF == 1) {
            // GLM's profile ends with each live slot's own finished output, f32 [row-slot][hidden]: four slots a wave,
            // every load of the four in flight together, nothing to add up
            for (uint32_t k0 = 0; k0 < kt; k0 += 16u) {
                SlotRef sk[kMine];
                uint32_t qk[kMine];
                float v[kMine][2];
#pragma unroll
                for (uint32_t r = 0; r < kMine; ++r) {
                    const uint32_t k = k0 + NW * r + sg;
                    const uint32_t info = k < kt ? cinfo[k] : 0xFFFFFFFFu;
                    sk[r].row = s.row;
                    sk[r].live = info != 0xFFFFFFFFu;
                    sk[r].shared = false;
                    sk[r].e = info & 0x7FFFFFFFu;
                    qk[r] = s.row * kt + (k < kt ? k : 0u);
                }
                routed_down_finish_many<true, XLDS, kMine, 1, kDefer>(a, sk, qk, b128, lane, v, ks);
#pragma unroll
                for (uint32_t r = 0; r < kMine; ++r)
                    if (sk[r].live) {
                        float* o = static_cast<float*>(a.y) + static_cast<size_t>(qk[r]) * a.hidden + b128 * 128u + lane;
                        o[0] = v[r][0];
                        o[64] = v[r][1];
                    }
            }
        } else {
            // The slots' finishes sixteen at a time, 16 / NW a wave with every load of a wave's slots in flight
            // together; wave 0 adds them in slot order.
            float(*fin)[128] = reinterpret_cast<float(*)[128]>(smem);
            float acc2[2] = {0.0f, 0.0f}, gated[2] = {0.0f, 0.0f};
            for (uint32_t k0 = 0; k0 < kt; k0 += 16u) {
                SlotRef sk[kMine];
                uint32_t qk[kMine];
                float v[kMine][2];
#pragma unroll
                for (uint32_t r = 0; r < kMine; ++r) {
                    const uint32_t k = k0 + NW * r + sg;
                    const uint32_t info = k < kt ? cinfo[k] : 0xFFFFFFFFu;
                    sk[r].row = s.row;
                    sk[r].live = info != 0xFFFFFFFFu;
                    sk[r].shared = sk[r].live && (info >> 31) != 0u;
                    sk[r].e = info & 0x7FFFFFFFu;
                    qk[r] = s.row * kt + (k < kt ? k : 0u);
                }
                if (finish_here) {  // the slots' workgroups finished them: their values, all in flight together
#pragma unroll
                    for (uint32_t r = 0; r < kMine; ++r) {
                        const float* zf = a.zd + static_cast<size_t>(qk[r]) * a.hidden + b128 * 128u;
                        v[r][0] = load_coherent(zf + lane);
                        v[r][1] = load_coherent(zf + lane + 64u);
                    }
                } else {
                    routed_down_finish_many<true, XLDS, kMine, 0, kDefer>(a, sk, qk, b128, lane, v, ks);
                }
#pragma unroll
                for (uint32_t r = 0; r < kMine; ++r)
                    if (sk[r].live) {
                        fin[NW * r + sg][lane] = v[r][0];
                        fin[NW * r + sg][lane + 64u] = v[r][1];
                    }
                __syncthreads();
                if (sg == 0u)
                    for (uint32_t w = 0; w < 16u && k0 + w < kt; ++w) {
                        if (cinfo[k0 + w] == 0xFFFFFFFFu) continue;
                        if (a.sigtab && (cinfo[k0 + w] >> 31) != 0u) {  // the gated shared expert's slot
                            gated[0] = gated_term(a, s.row, fin[w][lane]);
                            gated[1] = gated_term(a, s.row, fin[w][lane + 64u]);
                            continue;
                        }
                        const float wgt = cscore[k0 + w];
                        acc2[0] = __builtin_fmaf(wgt, fin[w][lane], acc2[0]);
                        acc2[1] = __builtin_fmaf(wgt, fin[w][lane + 64u], acc2[1]);
                    }
                __syncthreads();
            }
            if (sg == 0u) routed_store_row(a, s.row, b128, lane, acc2, gated);
        }
    }
}

template <int CB, int WIDE, int BT, int NPROJ, bool XLDS, bool ARRIVE, int PROF, int NW = 4>
__global__ void __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(WIDE ? 2 : (gemv_step_rows<CB>() == 2 ? 3 : 4)))) moe_gemv(const MoeLaunch a) {
    extern __shared__ __attribute__((aligned(16))) unsigned char xdyn[];
    __shared__ __attribute__((aligned(16))) unsigned char smem[NW * role_wave_lds_bytes<BT>()];
    __shared__ uint32_t last_flag, cinfo[64];
    __shared__ float cscore[64];
    gemv_role<CB, WIDE, BT, NPROJ, XLDS, ARRIVE, PROF, NW>(a, blockIdx.x, blockIdx.y, blockIdx.z, smem, xdyn, last_flag,
                                                           cinfo, cscore);
}

// ---- the grouped form ------------------------------------------------------------------------------------------
// Row-slots that read the same expert (or the same shared slot) are served by one set of workgroups: lane L's activation
// row of the matrix-core fragment is member L % 16's, so a tile decoded once multiplies up to sixteen rows. A column of
// the product depends on its own activation row alone, so a member's sums are the ones it gets alone. Worth a launch of
// its own where the decode dominates the call (large experts at several rows).
constexpr uint32_t kGroupRows = 16u, kMaxRowSlots = 1024u;  // 16 rows x (top-k + shared slots <= 64)

// One workgroup, 256 threads. Members of a group in ascending row-slot order, groups in the order of their first member;
// an expert read more than sixteen times starts a new group. Three passes over the call's keys in LDS, four keys a read
// and the reads of a pass independent of one another (a first form with one dependent LDS read a step took 18 us at 128
// row-slots; this one 3 to 11 by the row-slots): a slot's rank among the slots of its key, the leaders before every slot,
// then each slot's leader and through it the group's index.
__global__ void __launch_bounds__(256) moe_group(const MoeLaunch a) {
    __shared__ __attribute__((aligned(16))) uint32_t key[kMaxRowSlots];
    __shared__ __attribute__((aligned(16))) uint32_t aux[kMaxRowSlots];  // rank, bit 31: leads a group
    __shared__ uint32_t pre[kMaxRowSlots];                               // leaders before the slot
    constexpr uint32_t kDead = 0xFFFFFFFFu;
    const uint32_t rkt = a.rows * (a.topk + a.shared_slots), n4 = (rkt + 3u) & ~3u;
    uint32_t* info = a.groups + 1;
    uint32_t* member = a.groups + 1u + 2u * rkt;
    for (uint32_t rk = threadIdx.x; rk < n4; rk += 256u) {
        uint32_t k = kDead;
        if (rk < rkt) {
            const SlotRef s = resolve_slot(a, rk);
            if (s.live) k = s.shared ? 0x80000000u | s.e : s.e;
        }
        key[rk] = k;
        aux[rk] = 0u;
    }
    __syncthreads();
    uint32_t total[4];  // rkt <= 1024: at most four slots a thread
#pragma unroll
    for (uint32_t it = 0; it < 4u; ++it) {
        const uint32_t rk = threadIdx.x + 256u * it;
        total[it] = 0u;
        if (rk >= rkt || key[rk] == kDead) continue;
        const uint32_t mine = key[rk];
        uint32_t before = 0, all = 0;
#pragma unroll 8
        for (uint32_t j = 0; j < n4; j += 4u) {
            const uint4v k4 = *reinterpret_cast<const uint4v*>(key + j);
#pragma unroll
            for (uint32_t c = 0; c < 4u; ++c) {
                const uint32_t m = k4[c] == mine ? 1u : 0u;
                all += m;
                before += j + c < rk ? m : 0u;
            }
        }
        total[it] = all;
        aux[rk] = before | (before % kGroupRows == 0u ? 0x80000000u : 0u);
    }
    __syncthreads();
#pragma unroll
    for (uint32_t it = 0; it < 4u; ++it) {
        const uint32_t rk = threadIdx.x + 256u * it;
        if (rk >= rkt) continue;
        uint32_t p = 0;
#pragma unroll 8
        for (uint32_t j = 0; j < n4; j += 4u) {
            const uint4v a4 = *reinterpret_cast<const uint4v*>(aux + j);
#pragma unroll
            for (uint32_t c = 0; c < 4u; ++c) p += j + c < rk ? a4[c] >> 31 : 0u;
        }
        pre[rk] = p;
    }
    __syncthreads();
#pragma unroll
    for (uint32_t it = 0; it < 4u; ++it) {
        const uint32_t rk = threadIdx.x + 256u * it;
        if (rk >= rkt || key[rk] == kDead) continue;
        const uint32_t mine = key[rk], rank = aux[rk] & 0x7FFFFFFFu;
        const uint32_t first = rank / kGroupRows * kGroupRows, pos = rank - first;
        uint32_t leader = rk;
        if (pos != 0u) {
#pragma unroll 8
            for (uint32_t j = 0; j < n4; j += 4u) {
                const uint4v k4 = *reinterpret_cast<const uint4v*>(key + j);
                const uint4v a4 = *reinterpret_cast<const uint4v*>(aux + j);
#pragma unroll
                for (uint32_t c = 0; c < 4u; ++c)  // rank `first` of this key leads (one slot of the call at most)
                    leader = k4[c] == mine && a4[c] == (first | 0x80000000u) ? j + c : leader;
            }
        }
        const uint32_t g = pre[leader];
        member[g * kGroupRows + pos] = rk;
        if (pos == 0u) {
            const uint32_t left = total[it] - first;
            info[2u * g] = mine;
            info[2u * g + 1u] = left < kGroupRows ? left : kGroupRows;
        }
    }
    if (threadIdx.x == 0u) a.groups[0] = rkt == 0u ? 0u : pre[rkt - 1u] + (aux[rkt - 1u] >> 31);
}

template <int BT>
constexpr uint32_t group_lds_bytes() {
    constexpr uint32_t stage = 4u * GemvStream<kMoeLdsRing, kMcg, kNarrow, 1, BT, XGlobal>::kStageBytes, red = 4u * kGroupRows * BT * 4u * 16u;
    return stage > red ? stage : red;
}

// Grid (out / 16 / BT, RKT * NPROJ, KS), 256 threads: workgroup row y serves group y / NPROJ (none past the table's count)
// as moe_gemv serves a row-slot, from the prepared rows of the five-launch form, z [KS][RKT][out] by member.
template <int CB, int WIDE, int BT, int NPROJ>
__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(WIDE ? 2 : (gemv_step_rows<CB>() == 2 ? 3 : 4)))) moe_gemv_grouped(const MoeLaunch a) {
    __shared__ __attribute__((aligned(16))) unsigned char smem[group_lds_bytes<BT>()];
    typedef GemvStream<kMoeLdsRing, CB, WIDE, 1, BT, XGlobal> StreamG;
    constexpr uint32_t kStage = StreamG::kStageBytes;
    const uint32_t g = blockIdx.y / NPROJ, proj = blockIdx.y % NPROJ, blk = blockIdx.x, ksl = blockIdx.z;
    if (g >= a.groups[0]) return;  // uniform over the workgroup
    const uint32_t rkt = a.rows * (a.topk + a.shared_slots);
    const uint32_t key = a.groups[1u + 2u * g], count = a.groups[2u + 2u * g];
    const uint32_t* member = a.groups + 1u + 2u * rkt + g * kGroupRows;
    const uint32_t sg = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), lane = threadIdx.x & 63u;
    const RoutedBank& bank = (key >> 31) != 0u ? a.shared : a.bank;
    const uint32_t e = key & 0x7FFFFFFFu;
    const uint32_t in = NPROJ == 2 ? a.hidden : a.inter, out = NPROJ == 2 ? a.inter : a.hidden;
    const uint32_t n = NPROJ == 2 ? a.n_gu : a.n_dn;
    const uint32_t per = NPROJ == 2 ? a.per_gu : a.per_dn, parts = NPROJ == 2 ? a.parts_gu : a.parts_dn;
    const uint32_t in_tiles = in >> 4, out_tiles = out >> 4, nw = n >> 1;
    const uint32_t* wmat = (NPROJ == 1 ? bank.down_t : (proj ? bank.up_t : bank.gate_t)) +
                           static_cast<size_t>(e) * in_tiles * out_tiles * nw;
    const uint32_t part = ksl * 4u + sg, tk0 = part * per;
    const uint64_t wstride = static_cast<uint64_t>(out_tiles) * nw;
    const uint32_t* wbase = wmat + static_cast<uint64_t>(blk) * BT * nw + tk0 * wstride;
    // the lane's activation row: member lane % 16's (a row past the members stays zero, its sums are dropped)
    const uint32_t m = lane & 15u;
    const uint32_t rk = member[m < count ? m : 0u];

    float4v acc[1][BT];
#pragma unroll
    for (int t = 0; t < BT; ++t) acc[0][t] = float4v{0.f, 0.f, 0.f, 0.f};
    if (part < parts) {  // uniform over the wave; a wave past the last part adds zeros below
        const uint32_t* xq = NPROJ == 1 ? a.hd : (proj ? a.xu : a.xg);
        constexpr int R = gemv_step_rows<CB>();
        constexpr uint32_t kIn = R == 1 ? 4u : 2u;  // bytes a prepared input (moe_gemv's XGlobal form)
        uint32_t xoff[1] = {x_frag_offset(lane, m < count, rk * in * kIn)};
        StreamG stream(
            wbase, static_cast<uint32_t>(wstride) * 4u, per, n, a.wbits,
            XGlobal{xq, static_cast<uint64_t>(rkt) * in * kIn, (tk0 / R) * 64u, 64u}, xoff, smem + sg * kStage, lane);
        stream.issue();
        stream.run(acc);
    }
    __syncthreads();
    float4v(*red)[kGroupRows][BT * 4] = reinterpret_cast<float4v(*)[kGroupRows][BT * 4]>(smem);
    if (m < count)
#pragma unroll
        for (int t = 0; t < BT; ++t) red[sg][m][t * 4 + (lane >> 4)] = acc[0][t];
    __syncthreads();
    float* z = NPROJ == 1 ? a.zd : (proj ? a.zu : a.zg);
    for (uint32_t idx = threadIdx.x; idx < count * (BT * 4u); idx += 256u) {
        const uint32_t mm = idx / (BT * 4u), i = idx % (BT * 4u), t = i >> 2;
        const float4v v = ((red[0][mm][i] + red[1][mm][i]) + red[2][mm][i]) + red[3][mm][i];
        float* dst = z + (static_cast<size_t>(ksl) * rkt + member[mm]) * out + (blk * BT + t) * 16u + 4u * (i & 3u);
        *reinterpret_cast<float4v*>(dst) = v;
    }
}

// Grid (inter / 128, RKT), 64 threads.
template <int PROF>
__global__ void __launch_bounds__(64) moe_mid(const MoeLaunch a) {
    routed_mid_block<false, false, PROF>(a, resolve_slot(a, blockIdx.y), blockIdx.y, blockIdx.x, threadIdx.x);
}

// Grid (hidden / 128, rows), 64 threads. PROF 1 (GLM's): the slots' own f32 outputs instead of their weighted sum.
template <int PROF>
__global__ void __launch_bounds__(64) moe_combine(const MoeLaunch a) {
    if constexpr (PROF == 0) routed_combine_block<false>(a, blockIdx.y, blockIdx.x, threadIdx.x);
    else routed_slots_block<false>(a, blockIdx.y, blockIdx.x, threadIdx.x);
}

template <int CB, int WIDE, int NPROJ, bool XLDS, bool ARRIVE, int PROF>
hipError_t launch_gemv_bt(const MoeLaunch& a, hipStream_t s) {
    const uint32_t out = NPROJ == 2 ? a.inter : a.hidden;
    const uint32_t bt = NPROJ == 2 ? a.bt_gu : a.bt_dn, ks = NPROJ == 2 ? a.ks_gu : a.ks_dn;
    const uint32_t rkt = a.rows * (a.topk + a.shared_slots);
    const size_t dyn_wave = XLDS ? ((NPROJ == 2 ? a.per_gu : a.per_dn) / gemv_step_rows<CB>() + 1u) * (kXldsRows * 64u) : 0u;
    if constexpr (NPROJ == 1 && ARRIVE) {
        // Both K slices of the down projection in one workgroup of eight waves (the host's rule: MoeLaunch::
        // dn_slices_a_wg): the kernel sees one slice and one plane. The launches behind their own stage launches keep a
        // workgroup a slice; the sums are added in the same order either way.
        if (ks == 2u && a.dn_slices_a_wg == 2u) {
            MoeLaunch b = a;
            b.ks_dn = 1u;
            const size_t dyn8 = 8u * dyn_wave;
            const dim3 grid8((out / 16u) / bt, rkt, 1u), block8(512);
            if constexpr (WIDE == kNarrow) {
                if (bt == 8u) {
                    hipLaunchKernelGGL((moe_gemv<CB, WIDE, 8, 1, XLDS, true, PROF, 8>), grid8, block8, dyn8, s, b);
                    return hipGetLastError();
                }
            }
            if (bt != 4u) return hipErrorInvalidValue;
            hipLaunchKernelGGL((moe_gemv<CB, WIDE, 4, 1, XLDS, true, PROF, 8>), grid8, block8, dyn8, s, b);
            return hipGetLastError();
        }
    }
    const dim3 grid((out / 16u) / bt, rkt * NPROJ, ks), block(256);
    const size_t dyn = 4u * dyn_wave;
    if constexpr (WIDE == kNarrow) {
        if (bt == 8u) {
            hipLaunchKernelGGL((moe_gemv<CB, WIDE, 8, NPROJ, XLDS, ARRIVE, PROF>), grid, block, dyn, s, a);
            return hipGetLastError();
        }
    }
    if (bt != 4u) return hipErrorInvalidValue;  // a wide rate's eight tiles never fit a load
    hipLaunchKernelGGL((moe_gemv<CB, WIDE, 4, NPROJ, XLDS, ARRIVE, PROF>), grid, block, dyn, s, a);
    return hipGetLastError();
}

// PROF 1 (GLM's roundings in the stages a launch runs itself) exists for the codebook forms a default or opt-in
// configuration serves: MCG's f16 weight, its pair form, and MUL1's deferred map
template <int NPROJ, bool XLDS, bool ARRIVE, int PROF = 0>
hipError_t launch_gemv_cb(const MoeLaunch& a, hipStream_t s) {
    return with_reader(NPROJ == 2 ? a.n_gu : a.n_dn, [&](auto reader) {
        constexpr int R = decltype(reader)::value;
        if constexpr (PROF == 0) {
            switch (a.codebook) {
                case kMul1: return launch_gemv_bt<kMul1, R, NPROJ, XLDS, ARRIVE, 0>(a, s);
                case kMcg: return launch_gemv_bt<kMcg, R, NPROJ, XLDS, ARRIVE, 0>(a, s);
                case kMul1Defer: return launch_gemv_bt<kMul1Defer, R, NPROJ, XLDS, ARRIVE, 0>(a, s);
                default: return launch_gemv_bt<kMcgPair, R, NPROJ, XLDS, ARRIVE, 0>(a, s);
            }
        } else {
            switch (a.codebook) {
                case kMul1Defer: return launch_gemv_bt<kMul1Defer, R, NPROJ, XLDS, ARRIVE, 1>(a, s);
                case kMcgPair: return launch_gemv_bt<kMcgPair, R, NPROJ, XLDS, ARRIVE, 1>(a, s);
                case kMcg: return launch_gemv_bt<kMcg, R, NPROJ, XLDS, ARRIVE, 1>(a, s);
                default: return hipErrorInvalidValue;
            }
        }
    });
}

template <int CB, int WIDE, int NPROJ>
hipError_t launch_grouped_bt(const MoeLaunch& a, hipStream_t s) {
    const uint32_t out = NPROJ == 2 ? a.inter : a.hidden;
    const uint32_t bt = NPROJ == 2 ? a.bt_gu : a.bt_dn, ks = NPROJ == 2 ? a.ks_gu : a.ks_dn;
    const uint32_t rkt = a.rows * (a.topk + a.shared_slots);
    const dim3 grid((out / 16u) / bt, rkt * NPROJ, ks), block(256);
    if constexpr (WIDE == kNarrow) {
        if (bt == 8u) {
            hipLaunchKernelGGL((moe_gemv_grouped<CB, WIDE, 8, NPROJ>), grid, block, 0, s, a);
            return hipGetLastError();
        }
    }
    if (bt != 4u) return hipErrorInvalidValue;
    hipLaunchKernelGGL((moe_gemv_grouped<CB, WIDE, 4, NPROJ>), grid, block, 0, s, a);
    return hipGetLastError();
}

template <int NPROJ>
hipError_t launch_grouped_cb(const MoeLaunch& a, hipStream_t s) {
    return with_reader(NPROJ == 2 ? a.n_gu : a.n_dn, [&](auto reader) {
        constexpr int R = decltype(reader)::value;
        switch (a.codebook) {
            case kMul1: return launch_grouped_bt<kMul1, R, NPROJ>(a, s);
            case kMcg: return launch_grouped_bt<kMcg, R, NPROJ>(a, s);
            case kMul1Defer: return launch_grouped_bt<kMul1Defer, R, NPROJ>(a, s);
            default: return launch_grouped_bt<kMcgPair, R, NPROJ>(a, s);
        }
    });
}

}  // namespace

hipError_t launch_moe_decode(const MoeLaunch& a, int form, hipStream_t s) {
    const uint32_t rkt = a.rows * (a.topk + a.shared_slots);
    hipError_t e;
    // Up to kMidInDownRows rows, every down wave runs the mid stage of its own 128-block first (the two launches hand
    // over at their boundary; the stage is run once a column workgroup). More rows: the gate|up launch's last arriver
    // at a block runs it once.
    const bool mid_in_down = a.rows <= kMidInDownRows;
    if (form == kMoeTwoLaunches && !a.glm) {
        if (a.stages & 1u)
            if ((e = mid_in_down ? launch_gemv_cb<2, true, false>(a, s) : launch_gemv_cb<2, true, true>(a, s)) != hipSuccess)
                return e;
        if (a.stages & 2u) return mid_in_down ? launch_gemv_cb<1, true, true>(a, s) : launch_gemv_cb<1, false, true>(a, s);
        return hipSuccess;
    }
    if (form == kMoeTwoLaunches && a.codebook != kMul1) {
        // GLM's profile in the same two launches (src/hip/plan.zig's form 9 under Profile.glm), its own roundings in the
        // stages the launches run themselves
        if ((e = mid_in_down ? launch_gemv_cb<2, true, false, 1>(a, s) : launch_gemv_cb<2, true, true, 1>(a, s)) != hipSuccess)
            return e;
        return mid_in_down ? launch_gemv_cb<1, true, true, 1>(a, s) : launch_gemv_cb<1, false, true, 1>(a, s);
    }
    if (form == kMoeGrouped) {
        // the five launches behind the grouping launch, either profile's stages around the grouped GEMVs
        hipLaunchKernelGGL(moe_group, dim3(1), dim3(256), 0, s, a);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        if (a.glm) hipLaunchKernelGGL(moe_prep<1>, dim3(a.hidden / 128u, rkt), dim3(64), 0, s, a);
        else hipLaunchKernelGGL(moe_prep<0>, dim3(a.hidden / 128u, rkt), dim3(64), 0, s, a);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        if ((e = launch_grouped_cb<2>(a, s)) != hipSuccess) return e;
        if (a.glm) hipLaunchKernelGGL(moe_mid<1>, dim3(a.inter / 128u, rkt), dim3(64), 0, s, a);
        else hipLaunchKernelGGL(moe_mid<0>, dim3(a.inter / 128u, rkt), dim3(64), 0, s, a);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        if ((e = launch_grouped_cb<1>(a, s)) != hipSuccess) return e;
        if (a.glm) hipLaunchKernelGGL(moe_combine<1>, dim3(a.hidden / 128u, a.rows), dim3(64), 0, s, a);
        else hipLaunchKernelGGL(moe_combine<0>, dim3(a.hidden / 128u, a.rows), dim3(64), 0, s, a);
        return hipGetLastError();
    }
    if (a.glm) {
        // GLM's profile on the five launches (MUL1 decoded weight by weight, or a configured decode_form): its own
        // roundings in the stages between the GEMVs
        hipLaunchKernelGGL(moe_prep<1>, dim3(a.hidden / 128u, rkt), dim3(64), 0, s, a);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        if ((e = launch_gemv_cb<2, false, false>(a, s)) != hipSuccess) return e;
        hipLaunchKernelGGL(moe_mid<1>, dim3(a.inter / 128u, rkt), dim3(64), 0, s, a);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        if ((e = launch_gemv_cb<1, false, false>(a, s)) != hipSuccess) return e;
        hipLaunchKernelGGL(moe_combine<1>, dim3(a.hidden / 128u, a.rows), dim3(64), 0, s, a);
        return hipGetLastError();
    }
    if (form == kMoeFiveLaunches) {
        hipLaunchKernelGGL(moe_prep<0>, dim3(a.hidden / 128u, rkt), dim3(64), 0, s, a);
        if ((e = hipGetLastError()) != hipSuccess) return e;
        if ((e = launch_gemv_cb<2, false, false>(a, s)) != hipSuccess) return e;
    } else {
        if ((e = launch_gemv_cb<2, true, false>(a, s)) != hipSuccess) return e;
    }
    hipLaunchKernelGGL(moe_mid<0>, dim3(a.inter / 128u, rkt), dim3(64), 0, s, a);
    if ((e = hipGetLastError()) != hipSuccess) return e;
    if ((e = launch_gemv_cb<1, false, false>(a, s)) != hipSuccess) return e;
    hipLaunchKernelGGL(moe_combine<0>, dim3(a.hidden / 128u, a.rows), dim3(64), 0, s, a);
    return hipGetLastError();
}


namespace {

// The softmax router of the gated shared expert's routed form (turboexl3 src/models/qwen38/kernels/shared/
// router_softmax_1..6.metal, a copy of the host's "mlxserve_moe_router_softmax"): a row's top-k experts by logit, ties
// to the lowest id, and their softmax weights renormalised over the k. The statements' order is the host kernel's: the
// softmax over all experts in f32; each selected weight rounded to the dtype; their total added up in ascending slot
// order in the dtype, rounding after every add; each weight divided by it and rounded. (The f32 sum over the experts is
// a wave reduction whose order no source fixes.) One wave a row: lane L holds experts L + 64 i, i < 32.
// Grid (rows), 64 threads.
//
// GATE: four more waves take the shared gate's logit of the row, x[row] . gate_vec in bf16, in the order the reference
// states for it (src/core/kernels/sources/gate_gemv.metal, gate_sum.metal: MLX's gemv at 2..4 rows): 8 groups of 32
// lanes, lane t of 256 adds the products of columns 4 t + 1024 i + {0, 1, 2, 3} in that order in f32 (a product of two
// bf16 values is exact in f32, so fused or not is the same sum), each group folds a shuffle-down tree (16, 8, 4, 2, 1),
// the 8 partials are added in group order, and the total rounds to bf16. Columns past `hidden` add nothing. 320 threads.
template <int DT, bool GATE>
__global__ void __launch_bounds__(GATE ? 320 : 64) route_softmax(const void* logits, int32_t* inds, void* scores,
                                                                 uint32_t experts, uint32_t k, const uint16_t* gx,
                                                                 const uint16_t* gw, uint16_t* glogit, uint32_t hidden) {
    const uint32_t row = blockIdx.x, lane = threadIdx.x & 63u;
    if constexpr (GATE) {
        __shared__ float gp[8];
        if (threadIdx.x >= 64u) {
            const uint32_t t = threadIdx.x - 64u;
            const uint16_t* xr = gx + static_cast<size_t>(row) * hidden;
            float res = 0.0f;
            for (uint32_t c = 4u * t; c < hidden; c += 1024u) {
                const uint2 xv = *reinterpret_cast<const uint2*>(xr + c), wv = *reinterpret_cast<const uint2*>(gw + c);
                res += bf16_value(static_cast<uint16_t>(xv.x)) * bf16_value(static_cast<uint16_t>(wv.x));
                res += bf16_value(static_cast<uint16_t>(xv.x >> 16)) * bf16_value(static_cast<uint16_t>(wv.x >> 16));
                res += bf16_value(static_cast<uint16_t>(xv.y)) * bf16_value(static_cast<uint16_t>(wv.y));
                res += bf16_value(static_cast<uint16_t>(xv.y >> 16)) * bf16_value(static_cast<uint16_t>(wv.y >> 16));
            }
#pragma unroll
            for (int off = 16; off >= 1; off >>= 1) res += __shfl_down(res, off, 32);
            if ((t & 31u) == 0u) gp[t >> 5] = res;
        }
        __syncthreads();
        if (threadIdx.x == 64u) {
            float total = gp[0];
            for (uint32_t g = 1; g < 8u; ++g) total += gp[g];
            glogit[row] = bf16_bits(total);
        }
        if (threadIdx.x >= 64u) return;
    }
    const size_t base = static_cast<size_t>(row) * experts;
    constexpr float kNone = -__builtin_inff();
    float mine[32];
#pragma unroll
    for (uint32_t i = 0; i < 32u; ++i) {
        const uint32_t e = lane + 64u * i;
        mine[i] = e < experts ? load_act<DT>(logits, base + e) : kNone;
    }
    auto wave_max = [](float v) {
#pragma unroll
        for (int m = 32; m > 0; m >>= 1) v = fmaxf(v, __shfl_xor(v, m, 64));
        return v;
    };
    float lane_max = kNone;
#pragma unroll
    for (uint32_t i = 0; i < 32u; ++i) lane_max = fmaxf(lane_max, mine[i]);
    const float smax = wave_max(lane_max);
    float sum = 0.0f;
#pragma unroll
    for (uint32_t i = 0; i < 32u; ++i) sum += lane + 64u * i < experts ? __expf(mine[i] - smax) : 0.0f;
#pragma unroll
    for (int m = 32; m > 0; m >>= 1) sum += __shfl_xor(sum, m, 64);
    const float snorm = 1.0f / sum;

    auto round_dt = [](float v) {
        if constexpr (DT == kF16) return round_half(v);
        else if constexpr (DT == kBf16) return bf16_value(bf16_bits(v));
        else return v;
    };
    // k rounds of "max, then mask"
    uint32_t my_sel = 0;   // lane j < k keeps round j's pick
    float my_w = 0.0f;
    for (uint32_t r = 0; r < k; ++r) {
        float best = kNone;
        uint32_t slot = 0xFFFFFFFFu;
#pragma unroll
        for (uint32_t i = 0; i < 32u; ++i)
            if (mine[i] > best) {
                best = mine[i];
                slot = i;
            }
        const float gmax = wave_max(best);
        uint32_t cand = (best == gmax && slot != 0xFFFFFFFFu) ? lane + 64u * slot : 0xFFFFFFFFu;
#pragma unroll
        for (int m = 32; m > 0; m >>= 1) {
            const uint32_t o = static_cast<uint32_t>(__shfl_xor(static_cast<int>(cand), m, 64));
            cand = o < cand ? o : cand;
        }
        const uint32_t pick = cand < experts - 1u ? cand : experts - 1u;
        if ((pick & 63u) == lane) {
#pragma unroll
            for (uint32_t i = 0; i < 32u; ++i)
                if (i == pick >> 6) mine[i] = kNone;
        }
        if (lane == r) {
            my_sel = pick;
            my_w = round_dt(__expf(load_act<DT>(logits, base + pick) - smax) * snorm);
        }
    }
    float tot = 0.0f;
    for (uint32_t j = 0; j < k; ++j)
        tot = round_dt(__builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, my_w), static_cast<int>(j))) + tot);
    if (lane < k) {
        inds[static_cast<size_t>(row) * k + lane] = static_cast<int32_t>(my_sel);
        store_act<DT>(scores, static_cast<size_t>(row) * k + lane, my_w / round_dt(tot));
    }
}

}  // namespace

hipError_t launch_route_softmax(const void* logits, int32_t* inds, void* scores, uint32_t rows, uint32_t experts, uint32_t k,
                                int dtype, hipStream_t s) {
    const uint16_t* none = nullptr;
    uint16_t* out = nullptr;
    if (dtype == kF16) hipLaunchKernelGGL((route_softmax<kF16, false>), dim3(rows), dim3(64), 0, s, logits, inds, scores, experts, k, none, none, out, 0u);
    else if (dtype == kBf16) hipLaunchKernelGGL((route_softmax<kBf16, false>), dim3(rows), dim3(64), 0, s, logits, inds, scores, experts, k, none, none, out, 0u);
    else hipLaunchKernelGGL((route_softmax<kF32, false>), dim3(rows), dim3(64), 0, s, logits, inds, scores, experts, k, none, none, out, 0u);
    return hipGetLastError();
}

hipError_t launch_route_softmax_gate(const void* logits, int32_t* inds, void* scores, uint32_t rows, uint32_t experts,
                                     uint32_t k, const uint16_t* x, const uint16_t* gate_vec, uint16_t* glogit,
                                     uint32_t hidden, hipStream_t s) {
    hipLaunchKernelGGL((route_softmax<kBf16, true>), dim3(rows), dim3(320), 0, s, logits, inds, scores, experts, k, x,
                       gate_vec, glogit, hidden);
    return hipGetLastError();
}

}  // namespace t3
