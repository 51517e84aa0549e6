// `linear`: one dense EXL3 projection (turboexl3 src/root.zig:309-351), its chain form, and W_hat's decode.

#include <atomic>

#include "t3_host.hpp"

namespace t3 {
namespace {

struct DenseCall {
    DenseLaunch launch;
    size_t workspace = 0;
};

// root.linearOn's operand checks (src/root.zig:326-341), the loader's dtype rules (table/table.zig:129-145) and the
// dense plan's shape rule (src/hip/plan.zig:125-129).
int32_t check_dense(const t3_array* x, const t3_array* trellis, const t3_array* suh, const t3_array* svh,
                    t3_decode dec, const t3_array* y, uint32_t max_rows, DenseCall* call) {
    if (!array_ok(x) || !array_ok(trellis) || (suh && !array_ok(suh)) || (svh && !array_ok(svh)) || (y && !array_ok(y)))
        return T3_BadArgs;
    if (!aligned16(x) || !aligned16(trellis) || (suh && !aligned16(suh)) || (svh && !aligned16(svh)) || (y && !aligned16(y)))
        return T3_BadArgs;
    if (x->ndim < 1 || trellis->ndim != 3) return T3_BadExl3Shape;
    const int64_t in = trellis->shape[0] * 16, out = trellis->shape[1] * 16, n = trellis->shape[2];
    if (!rate_ok(n)) return T3_BadExl3Shape;
    if (in <= 0 || out <= 0 || in % 128 != 0 || out % 128 != 0 || in > (1ll << 30) || out > (1ll << 30))
        return T3_BadExl3Shape;
    if (x->shape[x->ndim - 1] != in) return T3_BadExl3Shape;
    if (suh && (suh->ndim < 1 || suh->shape[0] != in)) return T3_BadExl3Shape;
    if (svh && (svh->ndim < 1 || svh->shape[0] != out)) return T3_BadExl3Shape;
    if (!is_act_dtype(x->dtype)) return T3_BadExl3Dtype;
    if (trellis->dtype != T3_U16 && trellis->dtype != T3_I16) return T3_BadExl3Dtype;
    if ((suh && suh->dtype != T3_F16) || (svh && svh->dtype != T3_F16)) return T3_BadExl3Dtype;
    int64_t rows = 1;
    for (int i = 0; i + 1 < x->ndim; ++i) {
        rows *= x->shape[i];
        if (rows > (1ll << 30)) return T3_BadExl3Shape;
    }
    if (rows < 1) return T3_BadExl3Shape;
    if (y) {
        if (y->ndim != x->ndim || y->shape[y->ndim - 1] != out) return T3_BadExl3Shape;
        for (int i = 0; i + 1 < x->ndim; ++i)
            if (y->shape[i] != x->shape[i]) return T3_BadExl3Shape;
        if (y->dtype != x->dtype) return T3_BadExl3Dtype;
    }
    Dec d;
    if (const int32_t st = resolve_decode(dec, &d); st != T3_OK) return st;
    if (max_rows != 0 && rows > max_rows) return T3_Exl3EngineNotImplemented;
    // the kernels address one matrix, and one call's prepared rows, through 32-bit byte offsets
    if ((in / 16) * (out / 16) * n * 2 >= (1ll << 31) || rows * in * 4 >= (1ll << 31)) return T3_Exl3EngineNotImplemented;
    if (!widths_served(in, out) || !rows_served(rows, in, out)) return T3_Exl3EngineNotImplemented;
    if (out / 128 > static_cast<int64_t>(kCounterBytes / 4)) return T3_Exl3EngineNotImplemented;

    DenseLaunch& l = call->launch;
    l.x = x->data;
    l.suh = suh ? static_cast<const uint16_t*>(suh->data) : nullptr;
    l.svh = svh ? static_cast<const uint16_t*>(svh->data) : nullptr;
    l.trellis = static_cast<const uint32_t*>(trellis->data);
    l.y = y ? y->data : nullptr;
    l.in = static_cast<uint32_t>(in);
    l.out = static_cast<uint32_t>(out);
    l.rows = static_cast<uint32_t>(rows);
    l.n = static_cast<uint32_t>(n);
    l.wbits = d.wbits;
    l.codebook = d.gemv_form;
    l.dtype = x->dtype;
    dense_gemv_partition(l.n, l.in, l.out, &l.bt, &l.ks);
    return T3_OK;
}

// arrival counters u32 [out / 128] (fixed place), xq u32 [in / 16][rows][16], xs f32 [rows][in / 128], z f32 [ks][rows][out]
void carve_dense(DenseCall* call, void* workspace) {
    DenseLaunch& l = call->launch;
    Carver c(workspace);
    l.arrive = c.take<uint32_t>(kCounterBytes);
    l.xq = c.take<uint32_t>(static_cast<size_t>(l.rows) * l.in * 4u);
    // the one-launch form keeps a copy of the block sums a 128-column block (up to 4 rows)
    const size_t xs_copies = l.rows <= 4u ? l.out / 128u : 1u;
    l.xs = c.take<float>(xs_copies * l.rows * (l.in / 128u) * 4u);
    l.z = c.take<float>(static_cast<size_t>(l.ks) * l.rows * l.out * 4u);
    call->workspace = c.used;
}

// Above 32 rows: xq plain f16 [rows][in], xs f32 [rows][in / 128], z f32 [K parts][rows][out].
void carve_dense_prefill(DenseCall* call, void* workspace) {
    DenseLaunch& l = call->launch;
    l.ks = config().dense_rows_alone ? 1u : dense_prefill_kparts(l.rows, l.in, l.out);
    Carver c(workspace);
    l.arrive = c.take<uint32_t>(kCounterBytes);
    l.xq = c.take<uint32_t>(static_cast<size_t>(l.rows) * l.in * 2u);
    l.xs = c.take<float>(static_cast<size_t>(l.rows) * (l.in / 128u) * 4u);
    l.z = c.take<float>(static_cast<size_t>(l.ks) * l.rows * l.out * 4u);
    call->workspace = c.used;
}

constexpr uint32_t kGemvRowsMax = 32;
// The rows the GEMV serves in the configuration at hand. dense_rows_alone = 1 hands rows 17..32 to the trellis GEMM too:
// every row count above 16 then runs one kernel with one K order, and rows 0..16 of a 17-, 40-, 129- or 200-row call
// share their bytes as the reference's own GEMM holds them (src/hip_tests.zig:866-880).
uint32_t gemv_rows_max() { return config().dense_rows_alone ? 16u : kGemvRowsMax; }

// From dense_gemm_rows rows up a dense call decodes W_hat once and multiplies plainly (src/core/dense.zig:909-922,
// 1290-1302): the decode is paid once a call, not once a 128-row item, and the plain GEMM shares K out where its tiles are
// few (gemm_kparts), so it fills the GPU at any shape. Measured over ten model shapes x eight row counts from 256 to 4096
// (trellis GEMM against W_hat form, us): up to 512 rows (four items) the trellis GEMM wins or ties everywhere (4096 x 4096
// 47 / 63, 4096 x 14336 98 / 109); from five items on the W_hat form does (640 rows: 4096 x 4096 64 / 56, 4096 x 14336
// 158 / 130, 14336 x 4096 159 / 133, 7168 x 2048 60 / 55; 2048 rows: 2560 x 5120 109 / 84, 8192 x 8192 321 / 270), with
// ties at 1024 rows and two cells the other way (2048 x 2048 at 2048 rows 49 / 57, 7168 x 2048 at 1024 rows 65 / 75).
// Hence the default of 513.
bool takes_w_hat(const DenseLaunch& l) {
    const int32_t from = config().dense_gemm_rows;
    return !config().dense_rows_alone && from > 0 && l.rows >= static_cast<uint32_t>(from) && gemm_half_ok(l.in, l.out);
}

struct WhatScratch {
    uint16_t* w_hat;  // f16 [in][out]
    uint16_t* xp;     // f16 [rows][in], natural order
    float* planes;    // f32 [K parts][rows][out] where the GEMM shares K out (gemm_kparts > 1), else null
};

// the planes of the W_hat form's GEMM over few tiles
float* carve_gemm_planes(Carver& c, const DenseLaunch& l) {
    const uint32_t k = gemm_kparts(l.rows, l.in, l.out);
    return k > 1u ? c.take<float>(static_cast<size_t>(k) * l.rows * l.out * 4u) : nullptr;
}

WhatScratch carve_dense_w_hat(DenseCall* call, void* workspace) {
    DenseLaunch& l = call->launch;
    Carver c(workspace);
    l.arrive = c.take<uint32_t>(kCounterBytes);
    WhatScratch w;
    w.w_hat = c.take<uint16_t>(static_cast<size_t>(l.in) * l.out * 2u);
    w.xp = c.take<uint16_t>(static_cast<size_t>(l.rows) * l.in * 2u);
    w.planes = carve_gemm_planes(c, l);
    call->workspace = c.used;
    return w;
}

// prepare (natural order) -> finish(z = f16(xp W_hat)): the product and the finish are one launch, z stays in LDS; over
// few tiles the product's K is shared out into parts (planes) and the finish is a launch of its own
int32_t run_over_w_hat(const DenseLaunch& l, const uint16_t* w_hat, uint16_t* xp, float* planes, hipStream_t s) {
    if (const int32_t st = hip_status(launch_dense_prep_natural(l, xp, s)); st != T3_OK) return st;
    const uint32_t k = gemm_kparts(l.rows, l.in, l.out);
    if (k == 1u) return hip_status(launch_gemm_finish(xp, w_hat, l.svh, l.y, l.rows, l.in, l.out, l.dtype, s));
    if (!planes) return T3_BadArgs;
    if (const int32_t st = hip_status(launch_gemm_planes(xp, w_hat, planes, l.rows, l.in, l.out, l.out, 0u, false, k, s));
        st != T3_OK)
        return st;
    return hip_status(launch_dense_planes_finish(l, planes, k, s));
}

int32_t run_w_hat(const DenseCall& call, const WhatScratch& w, int codebook, hipStream_t s) {
    const DenseLaunch& l = call.launch;
    if (const int32_t st = hip_status(launch_dequant(l.trellis, w.w_hat, l.in, l.out, l.n, l.wbits, codebook, s));
        st != T3_OK)
        return st;
    return run_over_w_hat(l, w.w_hat, w.xp, w.planes, s);
}

// The operand checks of a call over a kept W_hat f16 [in, out]: `check_dense`'s, with the W_hat in the trellis's place.
int32_t check_resident(const t3_array* x, const t3_array* w_hat, const t3_array* suh, const t3_array* svh,
                       const t3_array* y, DenseCall* call) {
    if (!array_ok(x) || !array_ok(w_hat) || (suh && !array_ok(suh)) || (svh && !array_ok(svh)) || (y && !array_ok(y)))
        return T3_BadArgs;
    if (!aligned16(x) || !aligned16(w_hat) || (suh && !aligned16(suh)) || (svh && !aligned16(svh)) || (y && !aligned16(y)))
        return T3_BadArgs;
    if (x->ndim < 1 || w_hat->ndim != 2) return T3_BadExl3Shape;
    const int64_t in = w_hat->shape[0], out = w_hat->shape[1];
    if (in <= 0 || out <= 0 || in % 128 != 0 || out % 128 != 0 || in > (1ll << 30) || out > (1ll << 30))
        return T3_BadExl3Shape;
    if (x->shape[x->ndim - 1] != in) return T3_BadExl3Shape;
    if (suh && (suh->ndim < 1 || suh->shape[0] != in)) return T3_BadExl3Shape;
    if (svh && (svh->ndim < 1 || svh->shape[0] != out)) return T3_BadExl3Shape;
    if (!is_act_dtype(x->dtype) || w_hat->dtype != T3_F16) return T3_BadExl3Dtype;
    if ((suh && suh->dtype != T3_F16) || (svh && svh->dtype != T3_F16)) return T3_BadExl3Dtype;
    int64_t rows = 1;
    for (int i = 0; i + 1 < x->ndim; ++i) {
        rows *= x->shape[i];
        if (rows > (1ll << 30)) return T3_BadExl3Shape;
    }
    if (rows < 1) return T3_BadExl3Shape;
    if (y) {
        if (y->ndim != x->ndim || y->shape[y->ndim - 1] != out) return T3_BadExl3Shape;
        for (int i = 0; i + 1 < x->ndim; ++i)
            if (y->shape[i] != x->shape[i]) return T3_BadExl3Shape;
        if (y->dtype != x->dtype) return T3_BadExl3Dtype;
    }
    // decode and verify rows never read a W_hat (src/core/dense.zig:1309 `prefillOperands`)
    if (rows <= kGemvRowsMax || !gemm_half_ok(in, out)) return T3_Exl3EngineNotImplemented;
    if (rows * in * 4 >= (1ll << 31) || !widths_served(in, out) || !rows_served(rows, in, out)) return T3_Exl3EngineNotImplemented;
    DenseLaunch& l = call->launch;
    l.x = x->data;
    l.suh = suh ? static_cast<const uint16_t*>(suh->data) : nullptr;
    l.svh = svh ? static_cast<const uint16_t*>(svh->data) : nullptr;
    l.y = y ? y->data : nullptr;
    l.in = static_cast<uint32_t>(in);
    l.out = static_cast<uint32_t>(out);
    l.rows = static_cast<uint32_t>(rows);
    l.codebook = 1;  // an exact codebook (MCG's number): the W_hat holds finished weights, no deferred map
    l.dtype = x->dtype;
    l.ks = 1u;
    return T3_OK;
}

// arrival counters (untouched here: a workspace's head stays zero whoever is called with it), xp f16 [rows][in]
// (natural order)
void carve_resident(DenseCall* call, void* workspace, uint16_t** xp, float** planes) {
    DenseLaunch& l = call->launch;
    Carver c(workspace);
    l.arrive = c.take<uint32_t>(kCounterBytes);
    *xp = c.take<uint16_t>(static_cast<size_t>(l.rows) * l.in * 2u);
    *planes = carve_gemm_planes(c, l);
    call->workspace = c.used;
}

int32_t run_chain(const DenseCall& call, hipStream_t s, uint32_t stages) {
    if (stages & T3_STAGE_PREPARE)
        if (const int32_t st = hip_status(launch_dense_prep(call.launch, s)); st != T3_OK) return st;
    if (stages & T3_STAGE_GEMV)
        if (const int32_t st = hip_status(launch_dense_gemv(call.launch, kFuseChain, s)); st != T3_OK) return st;
    if (stages & T3_STAGE_FINISH) return hip_status(launch_dense_finish(call.launch, s));
    return T3_OK;
}

// The served form (src/core/dense.zig:1229-1242 takes DEC-ONE at its fewest rows the same way). Up to four rows where a
// wave takes eight tiles a step (up to four bits a weight), up to two otherwise: one launch where a wave's K part is whole
// 128-blocks and small enough to prepare in LDS, else the prepare launch and the arriving GEMV. More rows: the chain.
// Measured at 4096 x 12288 with the f16-weight codebook forms (us a call, one launch against the chain, four rows):
// K3 15.9-16.4 against 17.1, K4 16.4-16.5 against 17.0-17.2, K5 (four tiles a step) 17.9-18.1 against 17.6-17.7: every
// workgroup prepares every row of its K part (all rows' loads in flight together, then a butterfly a row) and the last
// arriver finishes a row a wave, which the chain's two small launches do once; with 16 and 32 rows the planes' coherent
// traffic costs the arriving form more than the finish launch it saves. The forms give the same bytes.
// (T3_ONE_ROWS_BT8, T3_ONE_ROWS_BT4: build-time overrides of the two bounds, for measuring.)
#ifndef T3_ONE_ROWS_BT8
#define T3_ONE_ROWS_BT8 4u
#endif
#ifndef T3_ONE_ROWS_BT4
#define T3_ONE_ROWS_BT4 2u
#endif
int dense_path(const DenseLaunch& l) {
    if (l.rows > gemv_rows_max()) return takes_w_hat(l) ? T3_DENSE_W_HAT_GEMM : T3_DENSE_TRELLIS_GEMM;
    const uint32_t per = (l.in / 16u) / (4u * l.ks);
    if (!config().dec_one || l.rows > (l.bt == 8u ? T3_ONE_ROWS_BT8 : T3_ONE_ROWS_BT4)) return T3_DENSE_CHAIN;
    return per % 8u == 0u && per <= 16u ? T3_DENSE_ONE_LAUNCH : T3_DENSE_ARRIVE;
}

int32_t run_fused(const DenseCall& call, hipStream_t s) {
    const DenseLaunch& l = call.launch;
    const int path = dense_path(l);
    if (path == T3_DENSE_CHAIN) return run_chain(call, s, 7u);
    if (path == T3_DENSE_ONE_LAUNCH) return hip_status(launch_dense_gemv(l, kFuseOne, s));
    if (const int32_t st = hip_status(launch_dense_prep(l, s)); st != T3_OK) return st;
    return hip_status(launch_dense_gemv(l, kFuseArrive, s));
}

}  // namespace
}  // namespace t3

extern "C" {

int32_t t3_linear_workspace_bytes(const t3_array* x, const t3_array* trellis, t3_decode dec, size_t* bytes) {
    const t3::ConfigScope one_config;
    if (!bytes) return T3_BadArgs;
    t3::DenseCall call;
    if (const int32_t st = t3::check_dense(x, trellis, nullptr, nullptr, dec, nullptr, 0, &call); st != T3_OK) return st;
    if (call.launch.rows > t3::gemv_rows_max() && t3::takes_w_hat(call.launch)) t3::carve_dense_w_hat(&call, nullptr);
    else if (call.launch.rows > t3::gemv_rows_max()) t3::carve_dense_prefill(&call, nullptr);
    else t3::carve_dense(&call, nullptr);
    *bytes = call.workspace;
    return T3_OK;
}

int32_t t3_linear_plan_of(const t3_array* x, const t3_array* trellis, t3_decode dec, t3_linear_plan* plan) {
    const t3::ConfigScope one_config;
    if (!plan) return T3_BadArgs;
    t3::DenseCall call;
    if (const int32_t st = t3::check_dense(x, trellis, nullptr, nullptr, dec, nullptr, 0, &call); st != T3_OK) return st;
    t3::DenseLaunch& l = call.launch;
    if (l.rows > t3::gemv_rows_max() && !t3::config().prefill) return T3_Exl3EngineNotImplemented;
    const int path = t3::dense_path(l);
    if (path == T3_DENSE_W_HAT_GEMM) t3::carve_dense_w_hat(&call, nullptr);
    else if (path == T3_DENSE_TRELLIS_GEMM) t3::carve_dense_prefill(&call, nullptr);
    else t3::carve_dense(&call, nullptr);
    t3_linear_plan p = {};
    p.path = path;
    p.rows = l.rows;
    p.in = l.in;
    p.out = l.out;
    p.n = l.n;
    p.code_bytes = static_cast<uint64_t>(l.in / 16u) * (l.out / 16u) * l.n * 2u;
    p.workspace_bytes = call.workspace;
    if (path <= T3_DENSE_CHAIN) {
        p.launches = path == T3_DENSE_ONE_LAUNCH ? 1 : path == T3_DENSE_ARRIVE ? 2 : 3;
        p.tiles_a_load = l.bt;
        p.k_slices = l.ks;
        p.tiles_a_wave = (l.in / 16u) / (4u * l.ks);
        p.workgroups = (l.out / 16u) / l.bt * l.ks;
    } else if (path == T3_DENSE_TRELLIS_GEMM) {
        p.launches = 3;
        p.k_slices = l.ks;  // carve_dense_prefill set the K parts
        const uint32_t item_rows = l.rows <= 64u ? 64u : 128u, items = (l.rows + item_rows - 1u) / item_rows;
        p.workgroups = t3::dense_prefill_workgroups(l.out, items) * l.ks;
    } else {
        // W_hat decode, prepare, the GEMM that finishes; over few tiles the GEMM's K parts and the finish by itself
        p.k_slices = t3::gemm_kparts(l.rows, l.in, l.out);
        p.launches = p.k_slices == 1u ? 3 : 4;
        p.workgroups = ((l.rows + 255u) / 256u) * ((l.out + 255u) / 256u) * p.k_slices;
    }
    *plan = p;
    return T3_OK;
}

int32_t t3_linear_chain(t3_stream stream, const t3_array* x, const t3_array* trellis, const t3_array* suh,
                        const t3_array* svh, t3_decode dec, t3_array* y, void* workspace, size_t workspace_bytes) {
    const t3::ConfigScope one_config;
    return t3_linear_stages(stream, x, trellis, suh, svh, dec, y, workspace, workspace_bytes,
                            T3_STAGE_PREPARE | T3_STAGE_GEMV | T3_STAGE_FINISH);
}

int32_t t3_linear_stages(t3_stream stream, const t3_array* x, const t3_array* trellis, const t3_array* suh,
                         const t3_array* svh, t3_decode dec, t3_array* y, void* workspace, size_t workspace_bytes,
                         uint32_t stages) {
    const t3::ConfigScope one_config;
    if (!suh || !svh || !y) return T3_BadArgs;
    if (stages == 0u || stages > 7u) return T3_BadArgs;
    t3::DenseCall call;
    if (const int32_t st = t3::check_dense(x, trellis, suh, svh, dec, y, 32, &call); st != T3_OK) return st;
    if (!t3::workspace_ok(workspace)) return T3_BadArgs;
    t3::carve_dense(&call, workspace);
    if (workspace_bytes < call.workspace) return T3_WorkspaceTooSmall;
    return t3::run_chain(call, static_cast<hipStream_t>(stream), stages);
}

int32_t t3_linear(t3_stream stream, const t3_array* x, const t3_array* trellis, const t3_array* suh,
                  const t3_array* svh, t3_decode dec, t3_array* y, void* workspace, size_t workspace_bytes) {
    const t3::ConfigScope one_config;
    if (!suh || !svh || !y) return T3_BadArgs;
    t3::DenseCall call;
    if (const int32_t st = t3::check_dense(x, trellis, suh, svh, dec, y, 0, &call); st != T3_OK) return st;
    if (!t3::workspace_ok(workspace)) return T3_BadArgs;
    if (call.launch.rows > t3::gemv_rows_max()) {
        if (!t3::config().prefill) return T3_Exl3EngineNotImplemented;
        if (t3::takes_w_hat(call.launch)) {
            const t3::WhatScratch w = t3::carve_dense_w_hat(&call, workspace);
            if (workspace_bytes < call.workspace) return T3_WorkspaceTooSmall;
            return t3::run_w_hat(call, w, dec.codebook, static_cast<hipStream_t>(stream));
        }
        // the trellis GEMM (the role of src/core/dense.zig:978-1034 and of dequant + matmul + finish, :909-922)
        t3::carve_dense_prefill(&call, workspace);
        if (workspace_bytes < call.workspace) return T3_WorkspaceTooSmall;
        return t3::hip_status(t3::launch_dense_prefill(call.launch, static_cast<hipStream_t>(stream)));
    }
    t3::carve_dense(&call, workspace);
    if (workspace_bytes < call.workspace) return T3_WorkspaceTooSmall;
    return t3::run_fused(call, static_cast<hipStream_t>(stream));
}

int32_t t3_linear_bias(t3_stream stream, const t3_array* x, const t3_array* trellis, const t3_array* suh,
                       const t3_array* svh, const t3_array* bias, t3_decode dec, t3_array* y, void* workspace,
                       size_t workspace_bytes) {
    const t3::ConfigScope one_config;
    // root.linearBias's own checks (src/root.zig:365-370), then `linear`, then one add in x's dtype
    if (!t3::array_ok(bias) || !t3::array_ok(trellis) || !t3::array_ok(x)) return T3_BadArgs;
    if (!t3::aligned16(bias)) return T3_BadArgs;
    if (trellis->ndim != 3 || bias->ndim != 1 || bias->shape[0] != trellis->shape[1] * 16) return T3_BadExl3Shape;
    if (bias->dtype != x->dtype) return T3_BadExl3Dtype;
    if (const int32_t st = t3_linear(stream, x, trellis, suh, svh, dec, y, workspace, workspace_bytes); st != T3_OK)
        return st;
    int64_t rows = 1;
    for (int i = 0; i + 1 < x->ndim; ++i) rows *= x->shape[i];
    return t3::hip_status(t3::launch_bias_add(y->data, bias->data, static_cast<uint32_t>(rows),
                                              static_cast<uint32_t>(bias->shape[0]), x->dtype,
                                              static_cast<hipStream_t>(stream)));
}

int32_t t3_dequant(t3_stream stream, const t3_array* trellis, t3_decode dec, t3_array* w_hat) {
    const t3::ConfigScope one_config;
    if (!t3::array_ok(trellis) || !t3::array_ok(w_hat)) return T3_BadArgs;
    if (!t3::aligned16(trellis) || !t3::aligned16(w_hat)) return T3_BadArgs;
    if (trellis->ndim != 3 || w_hat->ndim != 2) return T3_BadExl3Shape;
    const int64_t in = trellis->shape[0] * 16, out = trellis->shape[1] * 16, n = trellis->shape[2];
    if (!t3::rate_ok(n) || in <= 0 || out <= 0 || out % 64 != 0 || in > (1ll << 30) || out > (1ll << 30))
        return T3_BadExl3Shape;
    if (!t3::widths_served(in, out) || (in / 16) * (out / 16) * n * 2 >= (1ll << 32)) return T3_Exl3EngineNotImplemented;
    if (w_hat->shape[0] != in || w_hat->shape[1] != out) return T3_BadExl3Shape;
    if ((trellis->dtype != T3_U16 && trellis->dtype != T3_I16) || w_hat->dtype != T3_F16) return T3_BadExl3Dtype;
    t3::Dec d;
    if (const int32_t st = t3::resolve_decode(dec, &d); st != T3_OK) return st;
    return t3::hip_status(t3::launch_dequant(static_cast<const uint32_t*>(trellis->data),
                                             static_cast<uint16_t*>(w_hat->data), static_cast<uint32_t>(in),
                                             static_cast<uint32_t>(out), static_cast<uint32_t>(n), d.wbits, d.codebook,
                                             static_cast<hipStream_t>(stream)));
}

int32_t t3_linear_resident_workspace_bytes(const t3_array* x, const t3_array* w_hat, size_t* bytes) {
    const t3::ConfigScope one_config;
    if (!bytes) return T3_BadArgs;
    t3::DenseCall call;
    if (const int32_t st = t3::check_resident(x, w_hat, nullptr, nullptr, nullptr, &call); st != T3_OK) return st;
    uint16_t* xp;
    float* planes;
    t3::carve_resident(&call, nullptr, &xp, &planes);
    *bytes = call.workspace;
    return T3_OK;
}

int32_t t3_linear_resident(t3_stream stream, const t3_array* x, const t3_array* w_hat, const t3_array* suh,
                           const t3_array* svh, t3_array* y, void* workspace, size_t workspace_bytes) {
    const t3::ConfigScope one_config;
    if (!suh || !svh || !y) return T3_BadArgs;
    t3::DenseCall call;
    if (const int32_t st = t3::check_resident(x, w_hat, suh, svh, y, &call); st != T3_OK) return st;
    if (!t3::workspace_ok(workspace)) return T3_BadArgs;
    uint16_t* xp;
    float* planes;
    t3::carve_resident(&call, workspace, &xp, &planes);
    if (workspace_bytes < call.workspace) return T3_WorkspaceTooSmall;
    return t3::run_over_w_hat(call.launch, static_cast<const uint16_t*>(w_hat->data), xp, planes,
                              static_cast<hipStream_t>(stream));
}

int32_t t3_unrot_workspace_bytes(const t3_array* trellis, size_t* bytes) {
    const t3::ConfigScope one_config;
    if (!bytes || !t3::array_ok(trellis)) return T3_BadArgs;
    if (trellis->ndim != 3) return T3_BadExl3Shape;
    const int64_t in = trellis->shape[0] * 16, out = trellis->shape[1] * 16;
    if (in <= 0 || out <= 0) return T3_BadExl3Shape;
    t3::Carver c(nullptr);
    c.take<uint32_t>(t3::kCounterBytes);
    c.take<uint16_t>(static_cast<size_t>(in) * out * 2u);
    c.take<float>(static_cast<size_t>(in) * out * 4u);
    *bytes = c.used;
    return T3_OK;
}

int32_t t3_unrot_weight(t3_stream stream, const t3_array* trellis, const t3_array* suh, const t3_array* svh,
                        t3_decode dec, t3_array* w_std, int64_t col0, uint32_t* nonfinite, void* workspace,
                        size_t workspace_bytes) {
    const t3::ConfigScope one_config;
    if (!t3::array_ok(trellis) || !t3::array_ok(suh) || !t3::array_ok(svh) || !t3::array_ok(w_std) || !t3::workspace_ok(workspace))
        return T3_BadArgs;
    if (trellis->ndim != 3 || w_std->ndim != 2 || suh->ndim != 1 || svh->ndim != 1) return T3_BadExl3Shape;
    const int64_t in = trellis->shape[0] * 16, out = trellis->shape[1] * 16, n = trellis->shape[2];
    if (!t3::rate_ok(n) || in <= 0 || out <= 0 || in % 128 != 0 || out % 128 != 0 || in > (1ll << 30) ||
        out > (1ll << 30))
        return T3_BadExl3Shape;
    if (suh->shape[0] != in || svh->shape[0] != out || w_std->shape[0] != in || col0 < 0 || col0 % 8 != 0 ||
        col0 + out > w_std->shape[1] || w_std->shape[1] > (1ll << 30))
        return T3_BadExl3Shape;
    if ((trellis->dtype != T3_U16 && trellis->dtype != T3_I16) || suh->dtype != T3_F16 || svh->dtype != T3_F16 ||
        (w_std->dtype != T3_F16 && w_std->dtype != T3_BF16))
        return T3_BadExl3Dtype;
    if (!t3::aligned16(trellis) || !t3::aligned16(suh) || !t3::aligned16(svh) || !t3::aligned16(w_std) ||
        w_std->shape[1] % 8 != 0)
        return T3_BadArgs;
    if (!t3::widths_served(in, out) || in * out >= (1ll << 32) || (in / 16) * (out / 16) * n * 2 >= (1ll << 32))
        return T3_Exl3EngineNotImplemented;
    t3::Dec d;
    if (const int32_t st = t3::resolve_decode(dec, &d); st != T3_OK) return st;
    t3::Carver c(workspace);
    c.take<uint32_t>(t3::kCounterBytes);  // a workspace's head: the fused launches' counters, left alone
    uint16_t* w_hat = c.take<uint16_t>(static_cast<size_t>(in) * out * 2u);
    float* r = c.take<float>(static_cast<size_t>(in) * out * 4u);
    if (workspace_bytes < c.used) return T3_WorkspaceTooSmall;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (const int32_t st = t3::hip_status(t3::launch_dequant(static_cast<const uint32_t*>(trellis->data), w_hat,
                                                             static_cast<uint32_t>(in), static_cast<uint32_t>(out),
                                                             static_cast<uint32_t>(n), d.wbits, d.codebook, s));
        st != T3_OK)
        return st;
    return t3::hip_status(t3::launch_unrot(w_hat, r, static_cast<const uint16_t*>(suh->data),
                                           static_cast<const uint16_t*>(svh->data), w_std->data,
                                           static_cast<uint32_t>(in), static_cast<uint32_t>(out),
                                           static_cast<uint32_t>(w_std->shape[1]), static_cast<uint32_t>(col0),
                                           w_std->dtype, nonfinite, s));  // T3_F16, T3_BF16 = the kernels' numbering
}

namespace {
// the operand checks of a product over W_std; rows and in out
int32_t check_unrot(const t3_array* x, const t3_array* w_std, int64_t col0, int64_t cols, const t3_array* y, int64_t* rows_out,
                    int64_t* in_out) {
    if (!t3::array_ok(x) || !t3::array_ok(w_std) || (y && !t3::array_ok(y))) return T3_BadArgs;
    if (x->ndim < 1 || w_std->ndim != 2 || (y && y->ndim != x->ndim)) return T3_BadExl3Shape;
    const int64_t in = w_std->shape[0];
    int64_t rows = 1;
    for (int i = 0; i + 1 < x->ndim; ++i) {
        if (y && x->shape[i] != y->shape[i]) return T3_BadExl3Shape;
        rows *= x->shape[i];
    }
    if (x->shape[x->ndim - 1] != in || (y && y->shape[y->ndim - 1] != cols) || col0 < 0 || cols <= 0 ||
        col0 + cols > w_std->shape[1] || rows <= 0 || rows > (1ll << 30) || in > (1ll << 30) ||
        w_std->shape[1] > (1ll << 30))
        return T3_BadExl3Shape;
    if ((w_std->dtype != T3_F16 && w_std->dtype != T3_BF16) || x->dtype != w_std->dtype || (y && y->dtype != w_std->dtype))
        return T3_BadExl3Dtype;
    if (!t3::aligned16(x) || !t3::aligned16(w_std) || (y && !t3::aligned16(y)) || col0 % 8 != 0) return T3_BadArgs;
    if (rows <= 32 || !t3::gemm_half_ok(static_cast<uint64_t>(in), static_cast<uint64_t>(w_std->shape[1])))
        return T3_Exl3EngineNotImplemented;
    *rows_out = rows;
    *in_out = in;
    return T3_OK;
}
// K parts of the product over W_std: the W_hat form's, where the planes' four-column stores fit
uint32_t unrot_kparts(int64_t rows, int64_t in, int64_t cols) {
    if (cols % 4 != 0 || rows * cols >= (1ll << 31)) return 1u;
    return t3::gemm_kparts(static_cast<uint32_t>(rows), static_cast<uint32_t>(in), static_cast<uint32_t>(cols));
}
}  // namespace

int32_t t3_linear_unrot(t3_stream stream, const t3_array* x, const t3_array* w_std, int64_t col0, int64_t cols,
                        t3_array* y) {
    const t3::ConfigScope one_config;
    if (!y) return T3_BadArgs;
    int64_t rows = 0, in = 0;
    if (const int32_t st = check_unrot(x, w_std, col0, cols, y, &rows, &in); st != T3_OK) return st;
    return t3::hip_status(t3::launch_gemm_half(
        x->data, w_std->data, y->data, static_cast<uint32_t>(rows), static_cast<uint32_t>(in), static_cast<uint32_t>(cols),
        static_cast<uint32_t>(w_std->shape[1]), static_cast<uint32_t>(col0), w_std->dtype == T3_BF16,
        static_cast<hipStream_t>(stream)));
}

int32_t t3_linear_unrot_workspace_bytes(const t3_array* x, const t3_array* w_std, int64_t col0, int64_t cols, size_t* bytes) {
    const t3::ConfigScope one_config;
    if (!bytes) return T3_BadArgs;
    int64_t rows = 0, in = 0;
    if (const int32_t st = check_unrot(x, w_std, col0, cols, nullptr, &rows, &in); st != T3_OK) return st;
    t3::Carver c(nullptr);
    c.take<uint32_t>(t3::kCounterBytes);
    const uint32_t k = unrot_kparts(rows, in, cols);
    if (k > 1u) c.take<float>(static_cast<size_t>(k) * rows * cols * 4u);
    *bytes = c.used;
    return T3_OK;
}

int32_t t3_linear_unrot_parts(t3_stream stream, const t3_array* x, const t3_array* w_std, int64_t col0, int64_t cols,
                              t3_array* y, void* workspace, size_t workspace_bytes) {
    const t3::ConfigScope one_config;
    if (!y) return T3_BadArgs;
    int64_t rows = 0, in = 0;
    if (const int32_t st = check_unrot(x, w_std, col0, cols, y, &rows, &in); st != T3_OK) return st;
    if (!t3::workspace_ok(workspace)) return T3_BadArgs;
    t3::Carver c(workspace);
    c.take<uint32_t>(t3::kCounterBytes);  // the head stays as it is: the fused launches' counters
    const uint32_t k = unrot_kparts(rows, in, cols);
    float* planes = k > 1u ? c.take<float>(static_cast<size_t>(k) * rows * cols * 4u) : nullptr;
    if (workspace_bytes < c.used) return T3_WorkspaceTooSmall;
    const void* w = w_std->data;
    const uint32_t c0 = static_cast<uint32_t>(col0);
    const bool bf16 = w_std->dtype == T3_BF16;
    hipStream_t s = static_cast<hipStream_t>(stream);
    const uint32_t r = static_cast<uint32_t>(rows), i = static_cast<uint32_t>(in), n = static_cast<uint32_t>(cols);
    const uint32_t ldw = static_cast<uint32_t>(w_std->shape[1]);
    if (k == 1u) return t3::hip_status(t3::launch_gemm_half(x->data, w, y->data, r, i, n, ldw, c0, bf16, s));
    if (const int32_t st = t3::hip_status(t3::launch_gemm_planes(x->data, w, planes, r, i, n, ldw, c0, bf16, k, s)); st != T3_OK)
        return st;
    return t3::hip_status(t3::launch_gemm_planes_round(planes, y->data, r, n, k, bf16, s));
}

}  // extern "C"

/* ---- the decode-row projection for callers that cannot allocate ------------------------------------------------ */

namespace {

// The scratch `t3_linear` takes from its caller (arrival counters, prepared rows, block sums, planes), here in the
// library's own device memory: every GPU that runs this library holds its own copy of the array until the process
// ends. In host code the array's name is only a handle for hipGetSymbolAddress: the address each device gave its copy
// is looked up once a device and kept in `static_scratch_ptr`, and only that pointer ever reaches a kernel.
static __device__ __align__(256) unsigned char scratch[T3_STATIC_SCRATCH_BYTES];

constexpr int kMaxDevices = 64;
std::atomic<unsigned char*> static_scratch_ptr[kMaxDevices];

// grid (ceil(words / 256)), 256 threads
__global__ void __launch_bounds__(256) static_scratch_clear(uint32_t* p, uint32_t words) {
    const uint32_t i = blockIdx.x * 256u + threadIdx.x;
    if (i < words) p[i] = 0u;
}

int32_t static_scratch_clear_head(hipStream_t s, unsigned char* p) {
    const uint32_t words = static_cast<uint32_t>(t3::kCounterBytes / 4u);
    hipLaunchKernelGGL(static_scratch_clear, dim3((words + 255u) / 256u), dim3(256), 0, s, reinterpret_cast<uint32_t*>(p),
                       words);
    return hipGetLastError() == hipSuccess ? T3_OK : T3_HipFailed;
}

// The current device's copy of the array. The first call on a device looks its address up and clears the counter head
// on `s` (the loader zero-fills the array too; the clear makes the contract explicit). Two threads racing through the
// first call store the same address and both clear before their own launches on their own streams' order.
int32_t static_scratch_of(hipStream_t s, unsigned char** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return T3_HipFailed;
    unsigned char* p = static_scratch_ptr[dev].load(std::memory_order_acquire);
    if (!p) {
        void* sym = nullptr;
        if (hipGetSymbolAddress(&sym, HIP_SYMBOL(scratch)) != hipSuccess || !sym) return T3_HipFailed;
        p = static_cast<unsigned char*>(sym);
        if (static_scratch_clear_head(s, p) != T3_OK) return T3_HipFailed;
        static_scratch_ptr[dev].store(p, std::memory_order_release);
    }
    *out = p;
    return T3_OK;
}

}  // namespace

extern "C" {

int32_t t3_linear_static(t3_stream stream, const t3_array* x, const t3_array* trellis, const t3_array* suh,
                         const t3_array* svh, t3_decode dec, t3_array* y) {
    const t3::ConfigScope one_config;
    if (!suh || !svh || !y) return T3_BadArgs;
    t3::DenseCall call;
    if (const int32_t st = t3::check_dense(x, trellis, suh, svh, dec, y, 0, &call); st != T3_OK) return st;
    // decode rows only: above them `t3_linear` may run a library GEMM, which allocates
    if (call.launch.rows > t3::gemv_rows_max()) return T3_Exl3EngineNotImplemented;
    t3::carve_dense(&call, nullptr);
    if (call.workspace > static_cast<size_t>(T3_STATIC_SCRATCH_BYTES)) return T3_WorkspaceTooSmall;
    unsigned char* base = nullptr;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (const int32_t st = static_scratch_of(s, &base); st != T3_OK) return st;
    t3::carve_dense(&call, base);
    const int32_t st = t3::run_fused(call, s);
    // a launch that reported an error may have left part of the chain's counters counted: no caller can reach them
    if (st != T3_OK) static_scratch_clear_head(s, base);
    return st;
}

int32_t t3_linear_static_reset(t3_stream stream) {
    unsigned char* base = nullptr;
    hipStream_t s = static_cast<hipStream_t>(stream);
    if (const int32_t st = static_scratch_of(s, &base); st != T3_OK) return st;
    return static_scratch_clear_head(s, base);
}

}  // extern "C"
