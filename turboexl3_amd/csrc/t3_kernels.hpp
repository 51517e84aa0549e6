// Host-side launch descriptors of the kernel groups; the C ABI (t3_api.cpp) fills them after validation.
#pragma once

#include <hip/hip_runtime.h>

#include <cmath>
#include <cstddef>
#include <cstdint>

namespace t3 {

// One dense projection call. Buffers by role, as the reference's HIP plan names them (turboexl3
// src/hip/plan.zig:9-45): x, suh, svh, trellis, and the scratch xq (prepared rows), xs (block sums), z (planes).
struct DenseLaunch {
    const void* x = nullptr;
    const uint16_t* suh = nullptr;
    const uint16_t* svh = nullptr;
    const uint32_t* trellis = nullptr;
    uint32_t* xq = nullptr;
    float* xs = nullptr;
    float* z = nullptr;
    void* y = nullptr;
    uint32_t* arrive = nullptr;  // the fused launch's arrival counters
    uint32_t in = 0, out = 0, rows = 0, n = 0, wbits = 16;
    int codebook = 0;  // t3::Codebook
    int dtype = 0;     // t3::Dtype of x and y
    uint32_t ks = 1, bt = 4;
};

// the GEMV launch's form: 0 planes only (the chain), 1 + the finish by the last workgroup to arrive at a column block,
// 2 + the prepare inside the launch (up to 4 rows)
enum DenseFuse : int { kFuseChain = 0, kFuseArrive = 1, kFuseOne = 2 };

// Whether a dense GEMV whose waves walk `per` tile rows each takes its tiles through the direct-to-LDS ring (four rows'
// slots a wave) rather than the register ring: the LDS ring pays where a wave's walk is long (one row of 4096 x 151936,
// 64 tile rows a wave: the GEMV launch 4-6 % shorter at K3..K6) and costs a launch of 8 or 16 tile rows a wave 1-3 %.
// (T3_GEMV_LDS_RING_FROM: a build-time override for measuring one form everywhere; 0 also puts the routed GEMVs, whose
// waves walk eight tile rows, on the LDS ring.)
#ifndef T3_GEMV_LDS_RING_FROM
#define T3_GEMV_LDS_RING_FROM 32
#endif
inline bool dense_gemv_lds_ring(uint32_t per) { return per >= static_cast<uint32_t>(T3_GEMV_LDS_RING_FROM); }

hipError_t launch_dense_prep(const DenseLaunch& d, hipStream_t s);
hipError_t launch_dense_gemv(const DenseLaunch& d, int fuse, hipStream_t s);
hipError_t launch_dense_finish(const DenseLaunch& d, hipStream_t s);

// A bank of experts, expert e on axis 0 (turboexl3 src/root.zig:73-76): trellis [E][in/16][out/16][n] as u32 words,
// suh f16 [E][in], svh f16 [E][out]; gate, up: hidden -> inter; down: inter -> hidden.
struct RoutedBank {
    const uint32_t* gate_t = nullptr;
    const uint32_t* up_t = nullptr;
    const uint32_t* down_t = nullptr;
    const uint16_t* gate_suh = nullptr;
    const uint16_t* up_suh = nullptr;
    const uint16_t* down_suh = nullptr;
    const uint16_t* gate_svh = nullptr;
    const uint16_t* up_svh = nullptr;
    const uint16_t* down_svh = nullptr;
    uint32_t experts = 0;
};

// One routed call at decode rows. Scratch by the reference's role names (src/hip/plan.zig:29-39).
struct MoeLaunch {
    RoutedBank bank, shared;     // shared: the bank the shared slots read (shared_slots of its experts, in order)
    const void* x = nullptr;     // [rows][hidden] in dtype
    const int32_t* slots = nullptr;  // [rows][topk] expert ids
    const void* scores = nullptr;    // [rows][topk] in score_dt
    const void* shared_add = nullptr;  // moeWithShared: [rows][hidden] in dtype, or null
    // the gated shared expert (src/models/qwen38/api.zig:305-312): sigtab [65536] in dtype = the sigmoid of every 16-bit
    // pattern, slogit [rows] in dtype = the shared gate's logit; null: the shared slots are summed at weight 1
    const void* sigtab = nullptr;
    const void* slogit = nullptr;
    // GLM's rounding profile (src/hip/plan.zig:219-221): x bf16, y f32 [rows][topk][hidden] a slot, no scores
    int glm = 0;
    void* y = nullptr;
    uint32_t* arrive = nullptr;  // the two-launch form's arrival counters
    // the grouped form's table: [0] the number of groups; then {key, members} a group (key: the expert, bit 31 for a
    // shared slot); then 16 member row-slots a group. RKT groups at most.
    uint32_t* groups = nullptr;
    uint32_t* xg = nullptr;      // u32 [RKT][hidden]
    uint32_t* xu = nullptr;
    uint32_t* hd = nullptr;      // u32 [RKT][inter]
    float* sg = nullptr;         // f32 [RKT][hidden / 128]
    float* su = nullptr;
    float* hs = nullptr;         // f32 [RKT][inter / 128]
    float* xt = nullptr;         // above the decode rows, the deferred map: f32 [3][positions], a position's totals of
                                 // sg, su and hs for the GEMMs' ends
    float* zg = nullptr;         // f32 [ks_gu][RKT][inter]
    float* zu = nullptr;
    float* zd = nullptr;         // f32 [ks_dn][RKT][hidden]
    uint32_t hidden = 0, inter = 0, rows = 0, topk = 0, shared_slots = 0;
    uint32_t n_gu = 0, n_dn = 0, wbits = 16;
    uint32_t per_gu = 8, per_dn = 8, parts_gu = 0, parts_dn = 0, ks_gu = 1, ks_dn = 1, bt_gu = 8, bt_dn = 8;
    uint32_t dn_slices_a_wg = 1;  // K slices one workgroup of the served down launch holds (2: eight waves)
    int codebook = 0, dtype = 0, score_dt = 0, defer = 0;
    int pair_order = 0;  // decode rows: the GEMVs take two tile rows a step (the f16-weight codebook forms) and read their
                         // activations as plain f16 in pair-quad order; else one, doubled f16 in quad order
    float limit = 0.0f;
    int clamp_at = 0;  // format.ClampAt: 0 gate_in (the gate clamped before its SiLU), 1 silu_out (the SiLU's output)
    // prefill only (the route's roles, src/hip/plan.zig:40-45): row-slots sorted by expert. order [P] position ->
    // row-slot, inv [P] row-slot -> position (~0: skipped), items [max_items] {expert, first position, rows, 0},
    // counts [E + S + 4]: per-expert counts, then the item count and the placed total; cursor [E + S], a counter every
    // 32 words (a cache line each).
    uint32_t* order = nullptr;
    uint32_t* inv = nullptr;
    uint32_t* items = nullptr;
    uint32_t* counts = nullptr;
    uint32_t* cursor = nullptr;
    uint32_t max_items = 0, item_rows = 64;
    // which launches of the chain a call makes (t3_moe_stages: a profiler's or a benchmark's view of one stage at a
    // time; the workspace carries the stages' results between calls). Decode, two launches: bit 0 gate|up + mid, bit 1
    // down + combine. Prefill: bit 0 the route (clear, histogram, scan, place), 1 prepare, 2 gate|up GEMM, 3 mid, 4 down
    // GEMM, 5 combine. The other decode forms run whole.
    uint32_t stages = 0xFFFFFFFFu;
};

// Five launches (prepare, gate|up, mid, down, combine); four (each gate|up wave prepares its own 128-block in LDS);
// or two (gate|up + mid, down + combine: the last workgroup to arrive at a block runs the next stage). The same bytes.
// Or six: the five behind a grouping launch, the row-slots that read one expert served together (up to 16 a group), so
// the expert's tiles are decoded once for all of them. The same bytes again: an output column of the matrix core depends
// on its own activation row alone.
// Rows up to which the two-launch form runs the mid stage inside the down launch (every down wave for its own
// 128-block) and shapes both launches for few, long waves (t3_moe.hip)
constexpr uint32_t kMoeFewRows = 4;
// floats from one row-slot's block sums to the next in the down launch's own copies of them: whole 128-byte lines, so
// that the device-coherent stores of different slots never meet in a cache line
__host__ __device__ inline uint32_t hs_copy_stride(uint32_t inter) { return (inter / 128u + 31u) & ~31u; }
enum MoeForm : int { kMoeFiveLaunches = 0, kMoeFourLaunches = 1, kMoeTwoLaunches = 2, kMoeGrouped = 3 };
hipError_t launch_moe_decode(const MoeLaunch& a, int form, hipStream_t s);
// a row's top-k experts by logit (ties to the lowest id) and their renormalised softmax weights in the logits' dtype
hipError_t launch_route_softmax(const void* logits, int32_t* inds, void* scores, uint32_t rows, uint32_t experts, uint32_t k,
                                int dtype, hipStream_t s);
// the same launch with the shared gate's logit of every row beside it: glogit bf16 [rows] = x [rows][hidden] . gate_vec
hipError_t launch_route_softmax_gate(const void* logits, int32_t* inds, void* scores, uint32_t rows, uint32_t experts,
                                     uint32_t k, const uint16_t* x, const uint16_t* gate_vec, uint16_t* glogit,
                                     uint32_t hidden, hipStream_t s);

// Rows a GEMM item of a routed call of `slots` row-slots over `experts` experts (the shared slots' among them). An item
// pays its matrix's whole decode whatever its rows, so items are as tall as the experts' shares of the call: 32 rows
// when the mean share is small, 64, then a shape of eight row blocks once it passes 40. That shape runs with
// accumulators for all eight blocks (128-row items, two waves a SIMD) or for six (the route cuts items at 96 rows: three
// waves a SIMD, an item's decode and MFMAs about an eighth faster; 512 experts of 2560 x 640, 160 rows an expert: the
// call 2.11 -> 1.95 ms). The cut that costs fewer decodes wins: the items an expert becomes, 1 + P(rows > cut) +
// P(rows > 2 cut) + ..., with an expert's rows scattering around the mean share like sqrt(mean) (a uniform routing's
// counts), at 96 rows against 128, the 96-row count allowed the eighth its kernel is faster by. Mean 64: 96 (one item
// either way); 100-150: 128 (most experts one item instead of two); 160: 96 (two either way); 200: 128.
inline uint32_t moe_item_rows(size_t slots, size_t experts) {
#ifdef T3_MOE_ITEM_ROWS  // a build-time override, for measuring one shape everywhere
    return T3_MOE_ITEM_ROWS;
#endif
    const size_t share = slots / experts;
    if (share <= 24u) return 32u;
    if (share <= 40u) return 64u;
    const float mean = static_cast<float>(slots) / static_cast<float>(experts), sd = std::sqrt(mean);
    const auto items = [&](float cut) {
        float n = 1.0f;
        for (int j = 1; j <= 16; ++j) n += 0.5f * std::erfc((static_cast<float>(j) * cut - mean) / (sd * 1.41421356f));
        return n;
    };
    return items(96.0f) <= 1.12f * items(128.0f) ? 96u : 128u;
}

// The same call above the decode rows: route, prepare, gate|up GEMM, mid, down GEMM, combine. xg, xu, hd hold plain f16
// here (pair-quad order), zg, zu, zd one plane each, all by sorted position.
hipError_t launch_moe_prefill(const MoeLaunch& a, hipStream_t s);
// One dense projection above 32 rows: prepare (f16, pair-quad order), the trellis GEMM, finish. xq holds plain f16; ks = 1.
hipError_t launch_dense_prefill(const DenseLaunch& d, hipStream_t s);
// Its K parts (d.ks; z then holds that many planes, summed in part order by the finish): a call of few rows decodes the
// matrix once, and a workgroup per 256 columns alone would leave most of the GPU idle, so the tile rows are shared out
// while the launch stays within the workgroups the GPU holds at once. Each part keeps an even number of K = 32 steps, at
// least eight. Measured against the rule that grew the parts until the launch had at least 512 workgroups (us): 4096 x 4096
// at 300 / 640 / 1536 rows 59 / 78 / 113 -> 44 / 63 / 100, 2048 x 7168 at 512 / 1024 rows 64 / 82 -> 48 / 66, 4096 x 14336 at
// 128 / 256 / 512 rows 62 / 80 / 115 -> 45 / 61 / 100, 8192 x 8192 at 300 rows 107 -> 94.
inline uint32_t dense_prefill_kparts(uint32_t rows, uint32_t in, uint32_t out) {
    const uint32_t item_rows = rows <= 64u ? 64u : 128u, items = (rows + item_rows - 1u) / item_rows;
    const uint32_t nblk = (out + 255u) / 256u, steps = in / 32u;
    // the most parts that still fit one round of the 512 workgroups the GPU holds at once (two a compute unit): a launch
    // that spills into a second round takes that round's whole time for its few workgroups. (The 64-row item's smaller
    // accumulators would let four workgroups share a compute unit, but 1024 was measured slower than 512 for it as well:
    // 4096 x 14336 at 64 rows 39.3 against 32.2 us.)
    const uint32_t slots = 512u;
    uint32_t k = 1;
    while (k < 16u && steps % (4u * k) == 0u && steps / (2u * k) >= 8u && items * nblk * 2u * k <= slots) k *= 2u;
    return k;
}

// The trellis GEMM's grid over `nblk` workgroup columns (256 output columns each) and up to `max_items` items.
// Consecutive workgroup ids go round the eight dies, and an item's columns stay on `spread` of them (so the dies' L2s
// each hold few items' activations): with fewer than eight items an item's columns spread over 8, 4 or 2 dies, else
// they share one. Ids a die: nbs columns x the item groups.
inline uint32_t gemm_spread(uint32_t max_items) {
    uint32_t spread = 8u;
    while (spread > 1u && 8u / spread < max_items) spread >>= 1;
    return spread;
}
inline uint32_t gemm_grid_x(uint32_t nblk, uint32_t max_items) {
    const uint32_t spread = gemm_spread(max_items), nbs = (nblk + spread - 1u) / spread, group = 8u / spread;
    return 8u * nbs * ((max_items + group - 1u) / group);
}
// workgroups a K part of the dense trellis GEMM launches
inline uint32_t dense_prefill_workgroups(uint32_t out, uint32_t items) { return gemm_grid_x((out + 255u) / 256u, items); }

// The W_hat form's own prepare: natural order (plain f16 [rows][in], what a plain GEMM multiplies).
hipError_t launch_dense_prep_natural(const DenseLaunch& d, uint16_t* xp, hipStream_t s);

// The plain half-precision GEMM on the matrix cores (t3_gemm.hip): y [rows][cols] = x [rows][in] w[:, wcol0 : wcol0 + cols]
// for w [in][ldw] (the whole array: the kernel bounds its loads by the array's end), all f16 or all bf16, f32 accumulation,
// y row-contiguous. in a multiple of 32, ldw and wcol0 of 8, x and w 16-byte aligned, in * ldw * 2 under 4 GiB (gemm_half_ok).
hipError_t launch_gemm_half(const void* x, const void* w, void* y, uint32_t rows, uint32_t in, uint32_t cols, uint32_t ldw,
                            uint32_t wcol0, bool bf16, hipStream_t s);
// the same product over a W_hat with format.finishOutput at its end: y [rows][out] in `dtype` from the prepared rows
hipError_t launch_gemm_finish(const uint16_t* xp, const uint16_t* w_hat, const uint16_t* svh, void* y, uint32_t rows,
                              uint32_t in, uint32_t out, int dtype, hipStream_t s);
// The W_hat form over few tiles: the product's f32 sums a K part (planes f32 [kparts][rows][out]), then the finish over the
// planes summed in part order (the trellis GEMM's finish launch). A 256 x 256 tile a workgroup over the whole K leaves a
// call of few rows on a handful of compute units; K parts fill them.
hipError_t launch_gemm_planes(const void* x, const void* w, float* planes, uint32_t rows, uint32_t in, uint32_t cols,
                              uint32_t ldw, uint32_t wcol0, bool bf16, uint32_t kparts, hipStream_t s);
// the plain product's end over K parts: y [rows][cols] (f16 or bf16) = the planes summed in part order, one rounding
hipError_t launch_gemm_planes_round(const float* planes, void* y, uint32_t rows, uint32_t cols, uint32_t kparts, bool bf16,
                                    hipStream_t s);
hipError_t launch_dense_planes_finish(const DenseLaunch& d, const float* planes, uint32_t kparts, hipStream_t s);
// K parts of that GEMM: the most (a power of two, at most 16, each part at least 16 steps of K = 32) that keep the launch
// within one workgroup a compute unit; 1: the launch that ends with the finish itself. (Fewer parts where the planes are
// large, priced at 8 bytes an output a part through HBM, measured slower: the planes of such calls live in the Infinity
// Cache. 2048 x 7168 at 512 rows 50 -> 68 us, 2560 x 5120 at 1024 rows 63 -> 78.)
inline uint32_t gemm_kparts(uint32_t rows, uint32_t in, uint32_t out) {
    const uint32_t tiles = ((rows + 255u) / 256u) * ((out + 255u) / 256u), steps = in / 32u;
    uint32_t k = 1;
    while (k < 16u && tiles * 2u * k <= 256u && steps % (2u * k) == 0u && steps / (2u * k) >= 16u) k *= 2u;
    return k;
}
inline bool gemm_half_ok(uint64_t in, uint64_t ldw) {
    return in % 32u == 0u && ldw % 8u == 0u && in * ldw * 2u < (1ull << 32);
}

// y += bias in y's dtype (root.linearBias: one add after the projection's own output rounding)
hipError_t launch_bias_add(void* y, const void* bias, uint32_t rows, uint32_t out, int dtype, hipStream_t s);

// trellis [in/16][out/16][n] -> W_hat f16 [in][out], bit-exact (format.reconstructInner)
hipError_t launch_dequant(const uint32_t* trellis, uint16_t* w_hat, uint32_t in, uint32_t out, uint32_t n,
                          uint32_t wbits, int codebook, hipStream_t s);

// W_hat f16 [in][out] -> the un-rotated weight in `dtype` (f16 or bf16) at columns col0.. of w_std [in][ld]; r: f32
// [in][out] scratch; nonfinite: a counter of the weights that left the dtype's range (may be null)
hipError_t launch_unrot(const uint16_t* w_hat, float* r, const uint16_t* suh, const uint16_t* svh, void* w_std, uint32_t in,
                        uint32_t out, uint32_t ld, uint32_t col0, int dtype, uint32_t* nonfinite, hipStream_t s);

// test kernels: every codeword's MCG and MUL1 value and MUL1 byte sum; every tile's 256 codewords by code position
hipError_t launch_test_codebooks(uint16_t* mcg, uint16_t* mul1, uint16_t* t, hipStream_t s);
hipError_t launch_test_lane(const uint32_t* trellis, uint32_t n, uint32_t wbits, uint32_t tiles, uint16_t* cw,
                            uint16_t* mcg, uint16_t* mul1, hipStream_t s);
// test kernel: the kernels' f32 -> bf16 and f32 -> f16 narrowing and bf16 -> f32 widening of `count` values
hipError_t launch_test_convert(const float* in, uint16_t* bf16, uint16_t* f16, float* back, uint32_t count, hipStream_t s);
// test kernel: D = A B through the GEMV's MFMA with the fragments the kernels assume
hipError_t launch_test_mfma(const uint16_t* a, const uint16_t* b, float* d, hipStream_t s);
// measurement kernel: a plain 16-byte-a-lane read of `bytes` bytes (a multiple of 16) folded into sink [workgroups * 256]
hipError_t launch_test_hbm_read(const void* src, uint64_t bytes, uint32_t* sink, uint32_t workgroups, hipStream_t s);

}  // namespace t3
