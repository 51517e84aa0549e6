// Routed experts: `moe`, `moeClamped`, `moeWithShared` (turboexl3 src/root.zig:822-904,976-1004) and the fused
// shared-expert form, over the decode-row chain of t3_moe.hip.

#include "t3_host.hpp"

namespace t3 {
namespace {

struct MoeCall {
    MoeLaunch launch;
    size_t workspace = 0;
    int64_t rows = 0;
    size_t order_at = 0, inv_at = 0, items_at = 0, counts_at = 0;  // prefill: the route's arrays inside the workspace
};

// One projection's arrays against the geometry (src/root.zig:87-102).
int32_t check_proj(const t3_proj& p, int64_t experts, int64_t in, int64_t out, int64_t* n) {
    if (!array_ok(&p.trellis) || !array_ok(&p.suh) || !array_ok(&p.svh)) return T3_BadArgs;
    if (!aligned16(&p.trellis) || !aligned16(&p.suh) || !aligned16(&p.svh)) return T3_BadArgs;
    const t3_array& t = p.trellis;
    if (in <= 0 || out <= 0 || in % 128 != 0 || out % 128 != 0 || t.ndim != 4 || t.shape[0] != experts ||
        t.shape[1] != in / 16 || t.shape[2] != out / 16 || !rate_ok(t.shape[3]) || p.suh.ndim != 2 ||
        p.suh.shape[0] != experts || p.suh.shape[1] != in || p.svh.ndim != 2 || p.svh.shape[0] != experts ||
        p.svh.shape[1] != out)
        return T3_BadExl3Shape;
    if ((t.dtype != T3_U16 && t.dtype != T3_I16) || p.suh.dtype != T3_F16 || p.svh.dtype != T3_F16) return T3_BadExl3Dtype;
    *n = t.shape[3];
    return T3_OK;
}

// root.bankGeometry (src/root.zig:104-126): every projection validated; gate and up share a rate.
int32_t check_bank(const t3_bank* bank, int64_t hidden, RoutedBank* out, int64_t* inter, int64_t* n_gu, int64_t* n_dn) {
    if (!bank || !array_ok(&bank->gate.trellis)) return T3_BadArgs;
    const t3_array& g = bank->gate.trellis;
    if (g.ndim != 4 || g.shape[0] <= 0 || g.shape[2] <= 0 || g.shape[2] > (1 << 26)) return T3_BadExl3Shape;
    const int64_t experts = g.shape[0], width = g.shape[2] * 16;
    int64_t ng = 0, nu = 0, nd = 0;
    if (const int32_t st = check_proj(bank->gate, experts, hidden, width, &ng); st != T3_OK) return st;
    if (const int32_t st = check_proj(bank->up, experts, hidden, width, &nu); st != T3_OK) return st;
    if (const int32_t st = check_proj(bank->down, experts, width, hidden, &nd); st != T3_OK) return st;
    if (nu != ng) return T3_Exl3GateUpRateMismatch;
    // one expert's matrix is addressed through 32-bit byte offsets
    if ((hidden / 16) * (width / 16) * (ng > nd ? ng : nd) * 2 >= (1ll << 31)) return T3_Exl3EngineNotImplemented;
    out->gate_t = static_cast<const uint32_t*>(bank->gate.trellis.data);
    out->up_t = static_cast<const uint32_t*>(bank->up.trellis.data);
    out->down_t = static_cast<const uint32_t*>(bank->down.trellis.data);
    out->gate_suh = static_cast<const uint16_t*>(bank->gate.suh.data);
    out->up_suh = static_cast<const uint16_t*>(bank->up.suh.data);
    out->down_suh = static_cast<const uint16_t*>(bank->down.suh.data);
    out->gate_svh = static_cast<const uint16_t*>(bank->gate.svh.data);
    out->up_svh = static_cast<const uint16_t*>(bank->up.svh.data);
    out->down_svh = static_cast<const uint16_t*>(bank->down.svh.data);
    out->experts = static_cast<uint32_t>(experts);
    *inter = width;
    *n_gu = ng;
    *n_dn = nd;
    return T3_OK;
}

// root.validateCall (src/root.zig:128-141) and the partition of the decode chain.
int32_t check_moe(const t3_array* x, const t3_bank* bank, const t3_array* inds, const t3_array* scores,
                  const t3_bank* shared_bank, const t3_array* shared_add, t3_decode dec, int32_t limit,
                  const t3_array* y, MoeCall* call, int32_t clamp_at = 0) {
    if (!array_ok(x) || !array_ok(inds) || (scores && !array_ok(scores)) || (y && !array_ok(y)) ||
        (shared_add && !array_ok(shared_add)))
        return T3_BadArgs;
    if (!aligned16(x) || (y && !aligned16(y)) || (shared_add && !aligned16(shared_add))) return T3_BadArgs;
    if (x->ndim != 3 || inds->ndim != 3 || x->shape[0] <= 0 || x->shape[1] <= 0 || x->shape[0] != inds->shape[0] ||
        x->shape[1] != inds->shape[1] || inds->shape[2] <= 0 || inds->shape[2] > T3_REDUCE_MAX_TOPK)
        return T3_BadExl3Shape;
    if (x->shape[2] <= 0 || x->shape[2] % 128 != 0) return T3_BadExl3Shape;
    if (scores) {
        if (scores->ndim != 3) return T3_BadExl3Shape;
        for (int i = 0; i < 3; ++i)
            if (scores->shape[i] != inds->shape[i]) return T3_BadExl3Shape;
        if (!is_act_dtype(scores->dtype)) return T3_BadExl3Dtype;
    }
    if (!is_act_dtype(x->dtype) || (inds->dtype != T3_U32 && inds->dtype != T3_I32)) return T3_BadExl3Dtype;
    const int64_t rows = x->shape[0] * x->shape[1], topk = inds->shape[2], hidden = x->shape[2];
    if (rows > (1ll << 24) || rows * topk > (1ll << 28)) return T3_BadExl3Shape;
    MoeLaunch& l = call->launch;
    int64_t inter = 0, n_gu = 0, n_dn = 0;
    if (const int32_t st = check_bank(bank, hidden, &l.bank, &inter, &n_gu, &n_dn); st != T3_OK) return st;
    if (shared_bank) {
        int64_t s_inter = 0, s_gu = 0, s_dn = 0;
        if (const int32_t st = check_bank(shared_bank, hidden, &l.shared, &s_inter, &s_gu, &s_dn); st != T3_OK) return st;
        // the shared slots ride the routed launches: the same widths and rates
        if (s_inter != inter || s_gu != n_gu || s_dn != n_dn) return T3_Exl3EngineNotImplemented;
        if (topk + l.shared.experts > 64) return T3_BadExl3Shape;
        l.shared_slots = l.shared.experts;
    }
    if (shared_add) {
        if (shared_add->dtype != x->dtype) return T3_BadExl3Shape;  // src/root.zig:977
        int64_t count = 1;
        for (int i = 0; i < shared_add->ndim; ++i) count *= shared_add->shape[i];
        if (count != rows * hidden) return T3_BadExl3Shape;
    }
    if (y) {
        if (y->ndim != 3 || y->shape[0] != x->shape[0] || y->shape[1] != x->shape[1] || y->shape[2] != hidden)
            return T3_BadExl3Shape;
        if (y->dtype != x->dtype) return T3_BadExl3Dtype;
    }
    Dec d;
    if (const int32_t st = resolve_decode(dec, &d); st != T3_OK) return st;
    if (limit < 0 || limit > 128) return T3_InvalidExl3Clamp;
    call->rows = rows;
    l.x = x->data;
    l.slots = static_cast<const int32_t*>(inds->data);
    l.scores = scores ? scores->data : nullptr;
    l.score_dt = scores ? scores->dtype : T3_F32;
    l.shared_add = shared_add ? shared_add->data : nullptr;
    l.y = y ? y->data : nullptr;
    l.hidden = static_cast<uint32_t>(hidden);
    l.inter = static_cast<uint32_t>(inter);
    l.rows = static_cast<uint32_t>(rows);
    l.topk = static_cast<uint32_t>(topk);
    l.n_gu = static_cast<uint32_t>(n_gu);
    l.n_dn = static_cast<uint32_t>(n_dn);
    l.wbits = d.wbits;
    l.codebook = d.gemv_form;
    l.defer = d.gemv_form == 2;
    l.pair_order = d.gemv_form == 0 || d.gemv_form == 1;  // the f16-weight forms: two tile rows a GEMV step
    l.dtype = x->dtype;
    l.limit = static_cast<float>(limit);
    l.clamp_at = clamp_at;
    // Partitions: functions of the bank's shapes alone. gate|up: a part is one 128-block of the input (8 tiles), so a
    // wave can prepare its own block; down: the same (up to four rows a down wave runs the mid stage of its block
    // itself). Four tiles a down part were measured too: twice the workgroups of half the length, 2-5 % slower from three
    // rows up (8 tokens 63.5 against 62.0 us), because a down wave's 32 tiles are short against its launch's round trips.
    l.bt_gu = gemv_bt(l.n_gu);
    l.bt_dn = gemv_bt(l.n_dn);
    l.per_gu = 8;
    l.parts_gu = (l.hidden / 16u) / l.per_gu;
    l.ks_gu = (l.parts_gu + 3u) / 4u;
    l.per_dn = 8;
    l.parts_dn = (l.inter / 16u) / l.per_dn;
    l.ks_dn = (l.parts_dn + 3u) / 4u;
    // Up to kMoeFewRows rows the launches' waves are few and long against the call's chain of round trips: the gate|up
    // launch then takes four tiles a load (twice the workgroups of half the length; 512 experts of 2048 x 512 at one to
    // four tokens, the launch alone: 9.6 / 11.9 / 16.8 / 19.5 -> 8.2 / 11.4 / 15.7 / 18.8 us). The down launch keeps eight: its
    // workgroups count in at a counter a 128-column block, and twice the arrivals cost it more (one token 15.3 -> 15.8 us).
    // A column's sums do not depend on the tiles a load, so a row's bytes stay those of the row alone. (Where the gate|up
    // launch is small at eight tiles, within 2048 workgroups: large experts fill the GPU at one row already.)
    const uint64_t gu_wgs = static_cast<uint64_t>(l.inter / 128u) * l.rows * (l.topk + l.shared_slots) * 2u * l.ks_gu;
    if (l.rows <= kMoeFewRows && l.bt_gu == 8u && gu_wgs <= 2048u) l.bt_gu = 4u;
    // A down projection of two K slices (an intermediate size of 513 to 1024): the served launches hold both in one
    // workgroup of eight waves where those workgroups are resident all at once (two a CU): half the arrivals, no
    // second plane, and at eight tiles a load the workgroup finishes the slot's sums itself. The sums are added in the
    // planes' order, so the bytes are the chain's. Measured, a call, a workgroup a slice -> both in one: 512 experts of
    // 2560 x 640 top-10, MUL1 K3, one / two rows 28.5 -> 25.7 / 36.9 -> 34.1 us; MCG K4 27.0 -> 25.4 / 34.9 -> 33.8;
    // 2048 x 768 one / three rows 26.8 -> 25.2 / 41.0 -> 39.5. Past one round nothing is gained (the same shapes at
    // four rows 56.4 -> 56.4, 53.6 -> 54.4), nor where the experts are large (4096 x 1024: 39.4 -> 39.7).
    const uint64_t dn_wgs = static_cast<uint64_t>((l.hidden / 16u) / l.bt_dn) * l.rows * (l.topk + l.shared_slots);
    l.dn_slices_a_wg = l.ks_dn == 2u && dn_wgs <= 512u ? 2u : 1u;
    return T3_OK;
}

void carve_moe(MoeCall* call, void* workspace) {
    MoeLaunch& l = call->launch;
    const size_t rkt = static_cast<size_t>(l.rows) * (l.topk + l.shared_slots);
    Carver c(workspace);
    l.arrive = c.take<uint32_t>(kCounterBytes);
    l.xg = c.take<uint32_t>(rkt * l.hidden * 4u);
    l.xu = c.take<uint32_t>(rkt * l.hidden * 4u);
    l.hd = c.take<uint32_t>(rkt * l.inter * 4u);
    l.sg = c.take<float>(rkt * (l.hidden / 128u) * 4u);
    l.su = c.take<float>(rkt * (l.hidden / 128u) * 4u);
    // up to kMoeFewRows rows the down launch makes the sums itself: a copy a 128-column block of its output
    l.hs = c.take<float>(l.rows <= kMoeFewRows ? (l.hidden / 128u) * rkt * hs_copy_stride(l.inter) * 4u
                                               : rkt * (l.inter / 128u) * 4u);
    l.zg = c.take<float>(static_cast<size_t>(l.ks_gu) * rkt * l.inter * 4u);
    l.zu = c.take<float>(static_cast<size_t>(l.ks_gu) * rkt * l.inter * 4u);
    l.zd = c.take<float>(static_cast<size_t>(l.ks_dn) * rkt * l.hidden * 4u);
    l.groups = c.take<uint32_t>((1u + 2u * rkt + 16u * rkt) * 4u);  // the grouped form's table
    call->workspace = c.used;
}

// Above the decode rows every buffer is indexed by sorted position, the prepared activations are plain f16 and each
// projection has one plane; the route's arrays follow (src/hip/plan.zig:417-432 sizes the same roles).
void carve_moe_prefill(MoeCall* call, void* workspace) {
    MoeLaunch& l = call->launch;
    const size_t p = static_cast<size_t>(l.rows) * (l.topk + l.shared_slots);
    const size_t et = static_cast<size_t>(l.bank.experts) + l.shared_slots;
    l.item_rows = moe_item_rows(p, et);
    l.max_items = static_cast<uint32_t>((p < et ? p : et) + p / l.item_rows);
    Carver c(workspace);
    c.take<uint32_t>(kCounterBytes);
    l.xg = c.take<uint32_t>(p * l.hidden * 2u);
    l.xu = c.take<uint32_t>(p * l.hidden * 2u);
    l.hd = c.take<uint32_t>(p * l.inter * 2u);
    l.sg = c.take<float>(p * (l.hidden / 128u) * 4u);
    l.su = c.take<float>(p * (l.hidden / 128u) * 4u);
    l.hs = c.take<float>(p * (l.inter / 128u) * 4u);
    l.xt = c.take<float>(p * 3u * 4u);
    l.zg = c.take<float>(p * l.inter * 4u);
    l.zu = c.take<float>(p * l.inter * 4u);
    l.zd = c.take<float>(p * l.hidden * 4u);
    call->order_at = c.used;
    l.order = c.take<uint32_t>(p * 4u);
    call->inv_at = c.used;
    l.inv = c.take<uint32_t>(p * 4u);
    call->items_at = c.used;
    l.items = c.take<uint32_t>(static_cast<size_t>(l.max_items) * 16u);
    call->counts_at = c.used;
    l.counts = c.take<uint32_t>((et + 4u) * 4u);
    l.cursor = c.take<uint32_t>(et * 128u);  // a cache line a counter (t3_prefill.hip: kPfCounterStride)
    call->workspace = c.used;
}

// the rows a routed call takes through the GEMM chain, or the refusal (src/root.zig:850-853)
int32_t admit_prefill(const MoeCall& call) {
    if (!config().prefill) return T3_Exl3EngineNotImplemented;
    const MoeLaunch& l = call.launch;
    const int64_t p = static_cast<int64_t>(l.rows) * (l.topk + l.shared_slots);
    const int64_t widest = l.hidden > l.inter ? l.hidden : l.inter;
    // the GEMM addresses a projection's prepared rows through 32-bit byte offsets
    if (p * widest * 2 >= (1ll << 31)) return T3_Exl3EngineNotImplemented;
    return T3_OK;
}

// decode_form takes the reference's values (src/core/config.zig:8-12), every one with form 3's bytes there and here, each
// mapped to the form of this library that stands closest: 3 and 7 (the prepare a launch of its own): the five-launch
// chain; 5 and 6 ("share one decode among the row-slots that chose an expert"): the grouped six; 8 (the prepare inside
// the gate|up launch): four launches; 9: two launches while a counter a (row-slot, 128-block) fits the workspace's counter
// area (else four) and the gate|up launch stays within kTwoLaunchGroups workgroups (else the grouped six from two rows,
// the five at one).
// The two launches save three launch boundaries (~12 us of the chain) and pay with every gate|up workgroup's own prepare
// of its block (once a column workgroup instead of once) and the coherent hand-offs, ~8 % of the decode at eight tiles a
// load and twice that at four: past eight rounds of the GPU's resident workgroups the five launches are faster. Measured
// (two against five, us): 4096 x 2048 K4 top-8 at 4 / 5 / 8 / 16 rows 148.7 / 177.0 / 270.8 / 515.5 against 148.5 / 175.3 /
// 256.1 / 477.5; 7168 x 2048 K3 at 2 / 3 / 8 rows 131.9 / 189.0 / 449.4 against 133.9 / 180.1 / 415.6; 4096 x 1024 K5 at
// 4 / 8 rows 96.6 / 170.9 against 95.7 / 159.2; 2048 x 512 K3 top-10 at 16 rows 97.1 against 103.1. Past the bound the decode
// is what the call waits for, and serving the row-slots of one expert together pays (five against grouped, us: 4096 x 2048
// top-8 of 64 at 8 / 16 rows 256 / 468 against 208 / 274; eight experts of 4096 x 14336 top-2 at 16 rows 754 against 254).
// Every form gives the same bytes, so a row's bytes do not depend on which one its call took.
constexpr uint64_t kTwoLaunchGroups = 8192u;
int decode_form_of(const MoeLaunch& l) {
    const uint64_t rkt = static_cast<uint64_t>(l.rows) * (l.topk + l.shared_slots);
    const size_t widest = (l.hidden > l.inter ? l.hidden : l.inter) / 128u;
    const size_t counters = rkt * widest;
    const int32_t want = config().decode_form;
    if (want == 3 || want == 7) return kMoeFiveLaunches;
    if (want == 5 || want == 6) return kMoeGrouped;
    if (want == 8 || counters * 4u > kCounterBytes) return kMoeFourLaunches;
    // (workgroups at the rate's own tiles a load: the few-row calls' four tiles do not move the bound)
    const uint64_t gu_groups = static_cast<uint64_t>(l.inter / 16u / gemv_bt(l.n_gu)) * rkt * 2u * l.ks_gu;
    // where the decode dominates, the row-slots that read one expert are served together (a grouping launch in front):
    // every row-slot alone at worst, an expert's tiles decoded once for up to sixteen rows at best
    if (gu_groups > kTwoLaunchGroups) return l.rows >= 2u ? kMoeGrouped : kMoeFiveLaunches;
    // Below the bound the six launches cost ~20 us more of chain than the two, and win where grouping removes more decode
    // than that: by the groups a uniform routing is expected to leave (E (1 - (1 - k / E)^rows) experts hit, one group a
    // shared slot), gate|up workgroups saved = gu_groups (1 - groups / row-slots). Measured crossover ~1400 (two against
    // grouped, us: 128 experts of 2048 x 768 top-8 at 16 rows, 2200 saved, 108 / 96; 16 experts of 2048 x 1024 top-4 at 16
    // rows, 3100 saved, 68 / 49, at 8 rows, 1100 saved, 43 / 43; 512 of 2048 x 512 top-10 + shared at 16 rows, 1200 saved,
    // 100 / 106). A skewed routing groups better than this estimate.
    if (l.rows >= 2u) {
        const double e = static_cast<double>(l.bank.experts), k = static_cast<double>(l.topk);
        const double hit = e * (1.0 - __builtin_pow(1.0 - (k < e ? k / e : 1.0), static_cast<double>(l.rows)));
        const double groups = hit + static_cast<double>(l.shared_slots);
        const double saved = static_cast<double>(gu_groups) * (1.0 - groups / static_cast<double>(rkt));
        if (saved > 1400.0) return kMoeGrouped;
    }
    return kMoeTwoLaunches;
}

int32_t run_moe(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
                const t3_array* scores, const t3_bank* shared_bank, const t3_array* shared_add, t3_decode dec,
                int32_t limit, t3_array* y, void* workspace, size_t workspace_bytes, int32_t clamp_at = 0,
                uint32_t stages = 0xFFFFFFFFu) {
    if (!scores || !y) return T3_BadArgs;
    MoeCall call;
    if (const int32_t st = check_moe(x, bank, inds, scores, shared_bank, shared_add, dec, limit, y, &call, clamp_at);
        st != T3_OK)
        return st;
    call.launch.stages = stages;
    if (!workspace_ok(workspace)) return T3_BadArgs;
    // rows above the decode chain's take the prefill GEMM chain (src/root.zig:850-853)
    if (call.rows > T3_DECODE_ROWS_MAX) {
        if (const int32_t st = admit_prefill(call); st != T3_OK) return st;
        carve_moe_prefill(&call, workspace);
        if (workspace_bytes < call.workspace) return T3_WorkspaceTooSmall;
        return hip_status(launch_moe_prefill(call.launch, static_cast<hipStream_t>(stream)));
    }
    carve_moe(&call, workspace);
    if (workspace_bytes < call.workspace) return T3_WorkspaceTooSmall;
    return hip_status(launch_moe_decode(call.launch, decode_form_of(call.launch), static_cast<hipStream_t>(stream)));
}

}  // namespace
}  // namespace t3

extern "C" {

int32_t t3_moe_workspace_bytes(const t3_array* x, const t3_bank* bank, const t3_array* inds,
                               const t3_bank* shared_bank, size_t* bytes) {
    const t3::ConfigScope one_config;
    if (!bytes) return T3_BadArgs;
    t3::MoeCall call;
    const t3_decode dec = {0, 16};
    if (const int32_t st = t3::check_moe(x, bank, inds, nullptr, shared_bank, nullptr, dec, 0, nullptr, &call);
        st != T3_OK)
        return st;
    if (call.rows > T3_DECODE_ROWS_MAX) {
        if (const int32_t st = t3::admit_prefill(call); st != T3_OK) return st;
        t3::carve_moe_prefill(&call, nullptr);
    } else {
        t3::carve_moe(&call, nullptr);
    }
    *bytes = call.workspace;
    return T3_OK;
}

int32_t t3_moe_plan_of(const t3_array* x, const t3_bank* bank, const t3_array* inds, const t3_bank* shared_bank,
                       t3_moe_plan* plan) {
    const t3::ConfigScope one_config;
    if (!plan) return T3_BadArgs;
    t3::MoeCall call;
    const t3_decode dec = {0, 16};
    if (const int32_t st = t3::check_moe(x, bank, inds, nullptr, shared_bank, nullptr, dec, 0, nullptr, &call);
        st != T3_OK)
        return st;
    const t3::MoeLaunch& l = call.launch;
    t3_moe_plan p = {};
    p.rows = l.rows;
    p.row_slots = l.rows * (l.topk + l.shared_slots);
    p.hidden = l.hidden;
    p.inter = l.inter;
    p.topk = l.topk;
    p.shared_slots = l.shared_slots;
    p.expert_code_bytes = static_cast<uint64_t>(l.hidden / 16u) * (l.inter / 16u) * 2u * (2u * l.n_gu + l.n_dn);
    if (call.rows > T3_DECODE_ROWS_MAX) {
        if (const int32_t st = t3::admit_prefill(call); st != T3_OK) return st;
        t3::carve_moe_prefill(&call, nullptr);
        p.path = T3_MOE_PREFILL;
        p.launches = 9;
        p.item_rows = l.item_rows;
        p.max_items = l.max_items;
        p.route_order_at = call.order_at;
        p.route_inv_at = call.inv_at;
        p.route_items_at = call.items_at;
        p.route_counts_at = call.counts_at;
    } else {
        t3::carve_moe(&call, nullptr);
        const int form = t3::decode_form_of(l);
        p.path = form == t3::kMoeTwoLaunches ? T3_MOE_TWO_LAUNCHES
                 : form == t3::kMoeFourLaunches ? T3_MOE_FOUR_LAUNCHES
                 : form == t3::kMoeGrouped ? T3_MOE_GROUPED : T3_MOE_FIVE_LAUNCHES;
        p.launches = form == t3::kMoeTwoLaunches ? 2 : form == t3::kMoeFourLaunches ? 4 : form == t3::kMoeGrouped ? 6 : 5;
        p.tiles_a_wave_gu = l.per_gu;
        p.k_slices_gu = l.ks_gu;
        p.tiles_a_load_gu = l.bt_gu;
        p.tiles_a_wave_dn = l.per_dn;
        p.k_slices_dn = l.ks_dn;
        p.tiles_a_load_dn = l.bt_dn;
        p.k_slices_a_workgroup_dn = form == t3::kMoeTwoLaunches ? l.dn_slices_a_wg : 1u;
    }
    p.workspace_bytes = call.workspace;
    *plan = p;
    return T3_OK;
}

int32_t t3_moe(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
               const t3_array* scores, t3_decode dec, int32_t verify_rows, t3_array* y, void* workspace,
               size_t workspace_bytes) {
    const t3::ConfigScope one_config;
    (void)verify_rows;
    return t3::run_moe(stream, x, bank, inds, scores, nullptr, nullptr, dec, 0, y, workspace, workspace_bytes);
}

int32_t t3_moe_clamped(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
                       const t3_array* scores, t3_decode dec, int32_t limit, t3_array* y, void* workspace,
                       size_t workspace_bytes) {
    const t3::ConfigScope one_config;
    if (limit <= 0 || limit > 128) return T3_InvalidExl3Clamp;
    return t3::run_moe(stream, x, bank, inds, scores, nullptr, nullptr, dec, limit, y, workspace, workspace_bytes);
}

int32_t t3_moe_swiglu(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
                      const t3_array* scores, t3_decode dec, int32_t limit, int32_t clamp_at, t3_array* y,
                      void* workspace, size_t workspace_bytes) {
    const t3::ConfigScope one_config;
    if (limit < 0 || limit > 128 || (clamp_at != T3_CLAMP_GATE_IN && clamp_at != T3_CLAMP_SILU_OUT)) return T3_InvalidExl3Clamp;
    return t3::run_moe(stream, x, bank, inds, scores, nullptr, nullptr, dec, limit, y, workspace, workspace_bytes, clamp_at);
}

int32_t t3_moe_with_shared(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
                           const t3_array* scores, t3_decode dec, int32_t verify_rows, const t3_array* shared,
                           t3_array* y, void* workspace, size_t workspace_bytes) {
    const t3::ConfigScope one_config;
    (void)verify_rows;
    if (!shared) return T3_BadArgs;
    return t3::run_moe(stream, x, bank, inds, scores, nullptr, shared, dec, 0, y, workspace, workspace_bytes);
}

int32_t t3_moe_shared_expert(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
                             const t3_array* scores, t3_decode dec, int32_t limit, const t3_bank* shared_bank,
                             t3_array* y, void* workspace, size_t workspace_bytes) {
    const t3::ConfigScope one_config;
    if (!shared_bank) return T3_BadArgs;
    return t3::run_moe(stream, x, bank, inds, scores, shared_bank, nullptr, dec, limit, y, workspace, workspace_bytes);
}

int32_t t3_moe_stages(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
                      const t3_array* scores, t3_decode dec, int32_t limit, const t3_bank* shared_bank, t3_array* y,
                      void* workspace, size_t workspace_bytes, uint32_t stages) {
    const t3::ConfigScope one_config;
    if (limit < 0 || limit > 128) return T3_InvalidExl3Clamp;
    if (stages == 0u || stages > 63u) return T3_BadArgs;
    return t3::run_moe(stream, x, bank, inds, scores, shared_bank, nullptr, dec, limit, y, workspace, workspace_bytes, 0,
                       stages);
}

/* GLM's rounding profile of the routed experts (src/hip/plan.zig:219-247 `Profile.glm`): x bf16, each routed slot's own
 * f32 output, no scores; the slots of a row are the host's to combine. */
int32_t t3_moe_glm(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds, t3_decode dec,
                   int32_t limit, t3_array* y, void* workspace, size_t workspace_bytes) {
    const t3::ConfigScope one_config;
    if (!t3::array_ok(y)) return T3_BadArgs;
    if (limit < 0 || limit > 128) return T3_InvalidExl3Clamp;
    t3::MoeCall call;
    if (const int32_t st = t3::check_moe(x, bank, inds, nullptr, nullptr, nullptr, dec, limit, nullptr, &call, 0); st != T3_OK)
        return st;
    t3::MoeLaunch& l = call.launch;
    if (x->dtype != T3_BF16) return T3_BadExl3Shape;  // plan.zig:244
    if (y->dtype != T3_F32) return T3_BadExl3Dtype;
    if (y->ndim != 4 || y->shape[0] != x->shape[0] || y->shape[1] != x->shape[1] || y->shape[2] != inds->shape[2] ||
        y->shape[3] != x->shape[2] || !t3::aligned16(y))
        return T3_BadExl3Shape;
    if (!t3::workspace_ok(workspace)) return T3_BadArgs;
    l.y = y->data;
    l.glm = 1;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (call.rows > T3_DECODE_ROWS_MAX) {
        if (const int32_t st = t3::admit_prefill(call); st != T3_OK) return st;
        t3::carve_moe_prefill(&call, workspace);
        if (workspace_bytes < call.workspace) return T3_WorkspaceTooSmall;
        return t3::hip_status(t3::launch_moe_prefill(l, s));
    }
    t3::carve_moe(&call, workspace);
    if (workspace_bytes < call.workspace) return T3_WorkspaceTooSmall;
    // the four-launch form has no GLM statements of its own: the five launches stand in for it
    const int form = t3::decode_form_of(l);
    return t3::hip_status(t3::launch_moe_decode(l, form == t3::kMoeFourLaunches ? t3::kMoeFiveLaunches : form, s));
}

namespace {
// `moeFusedShared`; with `logits` [.., rows, E] and k, `moeFusedSharedRouted`: the slots and weights come from the
// router kernel, into the workspace's tail. bytes non-null: only the workspace size is wanted.
int32_t fused_shared(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
                     const t3_array* scores, const t3_array* logits, int64_t k, t3_decode dec, const t3_bank* shared_bank,
                     const t3_array* sigtab, const t3_array* logit, const t3_array* gate_vec, t3_array* y, void* workspace,
                     size_t workspace_bytes, size_t* bytes) {
    if (!shared_bank || !t3::array_ok(x)) return T3_BadArgs;
    t3_array routed_inds{}, routed_scores{};
    if (logits) {
        // src/models/qwen38/api.zig:396-407
        if (!t3::array_ok(logits)) return T3_BadArgs;
        if (x->ndim != 3 || logits->ndim != 3 || x->shape[0] != logits->shape[0] || x->shape[1] != logits->shape[1])
            return T3_BadExl3Shape;
        if (k <= 0 || k > 31 || logits->dtype != x->dtype || logits->shape[2] > 2048 || logits->shape[2] < k)
            return T3_Exl3EngineNotImplemented;
        routed_inds = *x;  // the shape [B, S, k]; the data pointer only has to be one until the workspace is carved
        routed_inds.dtype = T3_I32;
        routed_inds.shape[2] = k;
        routed_scores = routed_inds;
        routed_scores.dtype = x->dtype;
        inds = &routed_inds;
        scores = &routed_scores;
    }
    if (!scores) return T3_BadArgs;
    t3::MoeCall call;
    if (const int32_t st = t3::check_moe(x, bank, inds, scores, shared_bank, nullptr, dec, 0, bytes ? nullptr : y, &call, 0);
        st != T3_OK)
        return st;
    t3::MoeLaunch& l = call.launch;
    if (logits && logits->shape[2] != static_cast<int64_t>(l.bank.experts)) return T3_Exl3EngineNotImplemented;
    // what the fused launches do not carry stays with the caller's chain (src/models/qwen38/api.zig:312-322)
    if (call.rows > T3_SHARED_ROWS_MAX || l.shared_slots != 1u || (x->dtype != T3_F16 && x->dtype != T3_BF16))
        return T3_Exl3EngineNotImplemented;
    t3::carve_moe(&call, workspace);
    const size_t slots = static_cast<size_t>(call.rows) * l.topk;
    const size_t inds_at = call.workspace, scores_at = inds_at + ((slots * 4u + 255u) & ~static_cast<size_t>(255u));
    // the tail: slots, weights, and the shared gate's logit a row where the router's launch makes it
    const size_t glogit_at = scores_at + ((slots * 2u + 255u) & ~static_cast<size_t>(255u));
    const size_t total = logits ? glogit_at + 256u : call.workspace;
    if (bytes) {
        *bytes = total;
        return T3_OK;
    }
    if (!y || !t3::array_ok(sigtab)) return T3_BadArgs;
    // the logit, or (routed form only) the gate's vector: one of the two (src/models/qwen38/api.zig:399)
    if ((logit == nullptr) == (gate_vec == nullptr) || (gate_vec && !logits)) return T3_BadExl3Shape;
    int64_t tab = 1;
    for (int i = 0; i < sigtab->ndim; ++i) tab *= sigtab->shape[i];
    if (sigtab->dtype != x->dtype || tab != 65536) return T3_Exl3EngineNotImplemented;
    if (logit) {
        if (!t3::array_ok(logit)) return T3_BadArgs;
        int64_t lg = 1;
        for (int i = 0; i < logit->ndim; ++i) lg *= logit->shape[i];
        if (logit->dtype != x->dtype || lg != static_cast<int64_t>(call.rows)) return T3_Exl3EngineNotImplemented;
    } else {
        // the rows and widths MLX's matmul takes its 8-group gemv at (src/models/qwen38/api.zig:412-416)
        if (!t3::array_ok(gate_vec) || !t3::aligned16(gate_vec)) return T3_BadArgs;
        int64_t gv = 1;
        for (int i = 0; i < gate_vec->ndim; ++i) gv *= gate_vec->shape[i];
        const int64_t d = x->shape[2], rows = static_cast<int64_t>(call.rows);
        if (x->dtype != T3_BF16 || gate_vec->dtype != T3_BF16 || gv != d || rows < 2 || rows > 4 || d <= 64 || d < 16 * rows)
            return T3_Exl3EngineNotImplemented;
    }
    if (!t3::workspace_ok(workspace)) return T3_BadArgs;
    if (workspace_bytes < total) return T3_WorkspaceTooSmall;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (logits) {
        int32_t* d_inds = reinterpret_cast<int32_t*>(static_cast<unsigned char*>(workspace) + inds_at);
        void* d_scores = static_cast<unsigned char*>(workspace) + scores_at;
        uint16_t* d_glogit = reinterpret_cast<uint16_t*>(static_cast<unsigned char*>(workspace) + glogit_at);
        const uint32_t rows = static_cast<uint32_t>(call.rows);
        const hipError_t e =
            gate_vec ? t3::launch_route_softmax_gate(logits->data, d_inds, d_scores, rows, l.bank.experts, l.topk,
                                                     static_cast<const uint16_t*>(x->data),
                                                     static_cast<const uint16_t*>(gate_vec->data), d_glogit,
                                                     static_cast<uint32_t>(x->shape[2]), s)
                     : t3::launch_route_softmax(logits->data, d_inds, d_scores, rows, l.bank.experts, l.topk, x->dtype, s);
        if (const int32_t st = t3::hip_status(e); st != T3_OK) return st;
        l.slots = d_inds;
        l.scores = d_scores;
        l.score_dt = x->dtype;
        if (gate_vec) l.slogit = d_glogit;
    }
    l.sigtab = sigtab->data;
    if (logit) l.slogit = logit->data;
    return t3::hip_status(t3::launch_moe_decode(l, t3::decode_form_of(l), s));
}
}  // namespace

int32_t t3_moe_fused_shared(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
                            const t3_array* scores, t3_decode dec, const t3_bank* shared_bank, const t3_array* sigtab,
                            const t3_array* logit, t3_array* y, void* workspace, size_t workspace_bytes) {
    const t3::ConfigScope one_config;
    if (!inds || !scores || !y) return T3_BadArgs;
    if (!logit) return T3_BadArgs;
    return fused_shared(stream, x, bank, inds, scores, nullptr, 0, dec, shared_bank, sigtab, logit, nullptr, y, workspace,
                        workspace_bytes, nullptr);
}

int32_t t3_moe_fused_shared_routed_workspace_bytes(const t3_array* x, const t3_bank* bank, const t3_array* logits,
                                                   int64_t k, const t3_bank* shared_bank, size_t* bytes) {
    const t3::ConfigScope one_config;
    if (!bytes || !logits) return T3_BadArgs;
    const t3_decode dec = {0, 16};
    return fused_shared(nullptr, x, bank, nullptr, nullptr, logits, k, dec, shared_bank, nullptr, nullptr, nullptr, nullptr,
                        nullptr, 0, bytes);
}

int32_t t3_moe_fused_shared_routed(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* logits,
                                   int64_t k, t3_decode dec, const t3_bank* shared_bank, const t3_array* sigtab,
                                   const t3_array* logit, const t3_array* gate_vec, t3_array* y, void* workspace,
                                   size_t workspace_bytes) {
    const t3::ConfigScope one_config;
    if (!logits || !y) return T3_BadArgs;
    return fused_shared(stream, x, bank, nullptr, nullptr, logits, k, dec, shared_bank, sigtab, logit, gate_vec, y,
                        workspace, workspace_bytes, nullptr);
}

}  // extern "C"
