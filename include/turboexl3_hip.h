/*
 * turboexl3 on MI355X (gfx950): the C ABI of the EXL3 projection engine.
 *
 * Every entry point takes plain pointers, sizes and small POD descriptors; no C++ or framework types cross the
 * boundary. A descriptor (`t3_array`) stands where the reference passes an `mlx_array` handle: a device pointer
 * to row-contiguous data with its shape and dtype. Work is enqueued on the caller's HIP stream (`void*` =
 * `hipStream_t`, NULL = the null stream) and never synchronised here. Outputs and scratch are the caller's:
 * ask `*_workspace_bytes`, allocate once, pass the pointer. Inputs are borrowed, never copied or kept.
 *
 * Workspace contract: its first T3_WORKSPACE_COUNTER_BYTES bytes hold the arrival counters of the fused launches.
 * They must be zero when a workspace is first passed (zero-fill it once when you allocate it); every call leaves
 * them zero. Calls that share a workspace must be ordered on one stream: overlapping calls race on it. A call that
 * did not run to its end (a device error, a stream destroyed under it) may leave counters nonzero: zero-fill the
 * first T3_WORKSPACE_COUNTER_BYTES bytes again before the workspace is passed to another call.
 *
 * Refusal convention (turboexl3 docs/core/api.md:10-12): a call this library does not serve returns a named
 * status before it launches anything and leaves every output untouched; the caller runs its own chain.
 * The status names are the reference's Zig error names.
 *
 * Paths in comments are relative to the turboexl3 source tree.
 */
#ifndef TURBOEXL3_HIP_H
#define TURBOEXL3_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define T3_ABI_VERSION 4
#define T3_WORKSPACE_COUNTER_BYTES 65536

typedef void* t3_stream; /* hipStream_t */

/* ---- status ----------------------------------------------------------------------------------------------- */

typedef enum t3_status {
    T3_OK = 0,
    T3_BadExl3Shape = 1,                /* src/root.zig:93-101,128-141,309-326 */
    T3_BadExl3Dtype = 2,                /* src/root.zig:102,135-139,322 */
    T3_Exl3EngineNotImplemented = 3,    /* src/root.zig:841,851; docs/core/api.md:10-12 */
    T3_Exl3EngineCacheFull = 4,         /* src/root.zig:143-151 (kept for the name; this library has no cache to fill) */
    T3_Exl3GateUpRateMismatch = 5,      /* src/root.zig:117 */
    T3_InvalidExl3Clamp = 6,            /* src/root.zig:1002 */
    T3_Exl3TopKExceedsReduceBank = 7,   /* src/core/spec.zig:75-77 */
    T3_Exl3WindowUnsupported = 8,       /* src/core/spec.zig:49 */
    T3_ExpertLayoutUnsupported = 9,     /* src/core/spec.zig:38-48 */
    T3_InvalidTurboexl3Config = 10,     /* src/core/config.zig:175-178 */
    T3_WorkspaceTooSmall = 11,          /* this ABI: the caller's scratch is smaller than *_workspace_bytes says */
    T3_HipFailed = 12,                  /* src/hip/runtime.zig:6 */
    T3_BadArgs = 13,                    /* src/hip/runtime.zig:6: a null pointer or a descriptor that is not one */
    /* the quant table's names (table/config.zig:26, table/table.zig:128-174) */
    T3_NotExl3 = 14,
    T3_Exl3CodebookUnsupported = 15,
    T3_Exl3RateUnsupported = 16,
    T3_MissingWeight = 17,
    T3_Exl3TrellisGeometry = 18,
    T3_Exl3WidthNotMultipleOf128 = 19,
    T3_Exl3SideGeometry = 20,
    T3_Exl3SideDtype = 21
} t3_status;

/* The reference's error name of a status ("BadExl3Shape", ...); "ok" for T3_OK; never NULL. */
const char* t3_error_name(int32_t status);

/* ---- descriptors ------------------------------------------------------------------------------------------ */

typedef enum t3_dtype {
    T3_F32 = 0, T3_F16 = 1, T3_BF16 = 2, /* activations, scores (src/hip/plan.zig:72-73 numbering) */
    T3_U16 = 3, T3_I16 = 4,              /* trellis halfwords (src/root.zig:87-91) */
    T3_U32 = 5, T3_I32 = 6               /* expert ids (src/root.zig:136) */
} t3_dtype;

#define T3_MAX_DIMS 8

/* A row-contiguous device array: what an mlx_array handle carries for this path. Activations (x, y, an added shared
 * output), scale vectors and trellises start on a 16-byte boundary and a workspace on a 256-byte one (any allocation
 * or whole-row view does): the kernels read them 16 bytes a lane. T3_BadArgs otherwise. */
typedef struct t3_array {
    void* data;
    int32_t ndim;
    int32_t dtype; /* t3_dtype */
    int64_t shape[T3_MAX_DIMS];
} t3_array;

/* How a pack's trellis decodes (src/core/format.zig:71-78): codebook 0 = MUL1, 1 = MCG; window 8..16 bits. */
typedef struct t3_decode {
    int32_t codebook;
    int32_t window_bits;
} t3_decode;

/* One projection's arrays (src/root.zig:73-75): dense: trellis [in/16, out/16, n], suh [in], svh [out];
 * bank: a leading expert axis on each. trellis U16 or I16; suh, svh F16. */
typedef struct t3_proj {
    t3_array trellis, suh, svh;
} t3_proj;

typedef struct t3_bank {
    t3_proj gate, up, down;
} t3_bank;

/* ---- configuration (src/core/config.zig; only the fields this path reads) --------------------------------- */

typedef struct t3_config {
    int32_t decode_form;   /* the reference's values (src/core/config.zig:8-12: 3, 5, 6, 7, 8 or 9, each with form 3's bytes),
                            * mapped to this library's forms: 3, 7: the five-launch chain; 5, 6 (one decode shared among the
                            * row-slots that chose an expert): the grouped six launches whatever the size; 8: four launches
                            * (the prepare inside gate|up); 9 (default): two
                            * launches (mid and combine run by the last workgroup to arrive) while the gate|up launch
                            * stays within 8192 workgroups; past that (large experts at several rows, where the decode
                            * dominates), or where a uniform routing is expected to leave few enough experts hit, six: the
                            * five behind a grouping launch that serves the row-slots of one expert together; the same bytes
                            * whichever runs; others refused */
    int32_t dec_one;       /* 1 (default): dense decode rows in one launch; 0: the three-launch chain */
    int32_t prefill;       /* 1 (default); 0: routed calls above 16 rows refuse Exl3EngineNotImplemented */
    int32_t mcg_pair;      /* 0 (default): MCG's GEMV multiplies by the format's f16 weight (format.decodeMcg's bits), which holds
                            * the reference's bars at every shape; 1: it feeds the hashed pair to the matrix core unrounded
                            * (x lo + x hi in f32: this library's own form, ~5 % faster, inside the bars at the benchmark
                            * shapes and within 1.5 x of them on small random ones) */
    int32_t mul1_defer;    /* 1 (default): MUL1's affine map applied once an output (src/core/dense.zig deferFor); 0: per weight */
    int32_t dense_gemm_rows; /* dense calls of this many rows or more decode W_hat once into the workspace and run this
                              * library's plain f16 GEMM (K shared out over the grid where its tiles are few), which
                              * ends with the finish. Default 513: up to four 128-row items the trellis GEMM is the faster,
                              * from five on this form (measured over ten shapes); 0: never */
    int32_t dense_rows_alone; /* 0 (default): rows 17..32 run the GEMV and above 32 rows a dense call's launch shape follows
                               * its rows (K parts at few rows, the W_hat form at many), so a row's bytes can differ between
                               * calls of different row counts (each within the bars). 1: every call above 16 rows takes the
                               * trellis GEMM with one K part, and a row's bytes ignore the call's other rows, as the
                               * reference's own GEMM holds them for 17, 40, 129 and 200 rows (src/hip_tests.zig:866-880);
                               * few-row calls then run up to twice as long */
} t3_config;

/* The served configuration. */
void t3_config_default(t3_config* out);
/* Set once before the first call; a value this library does not serve returns T3_InvalidTurboexl3Config and
 * changes nothing (src/core/config.zig:175-178). */
int32_t t3_configure(const t3_config* cfg);
/* Kept for surface parity with src/root.zig:1148-1181: this library compiles nothing at run time and holds no
 * per-geometry state, so there is nothing to free. */
void t3_release_engines(void);

/* ---- dense projection (src/root.zig:309-351 `linear`) ------------------------------------------------------- */

/* y [..., out] in x's dtype for x [..., in]. Rows = the product of x's leading dims.
 * 1..32 rows: the trellis GEMV on the matrix cores; more: the trellis GEMM (weights decoded in registers), and from
 * t3_config.dense_gemm_rows rows: W_hat decoded once + a plain f16 GEMM. `y` is the caller's, shaped as x
 * with the last dim `out`. Status as root.linearOn's checks. */
int32_t t3_linear(t3_stream stream, const t3_array* x, const t3_array* trellis, const t3_array* suh,
                  const t3_array* svh, t3_decode dec, t3_array* y, void* workspace, size_t workspace_bytes);
/* Scratch bytes `t3_linear` needs for this call's shapes (the byte rules of src/hip/plan.zig:137-146 for this
 * library's own partition). */
int32_t t3_linear_workspace_bytes(const t3_array* x, const t3_array* trellis, t3_decode dec, size_t* bytes);

/* The three-launch chain of the same call (prepare, GEMV, finish): the chain `t3_linear`'s one launch must equal
 * byte for byte (src/core/gpu_test.zig:1016 holds DEC-ONE to the chain the same way). Rows 1..32 only. */
int32_t t3_linear_chain(t3_stream stream, const t3_array* x, const t3_array* trellis, const t3_array* suh,
                        const t3_array* svh, t3_decode dec, t3_array* y, void* workspace, size_t workspace_bytes);

/* `t3_linear_chain` with a choice of its launches, for profilers and hosts that bind the chain's roles themselves
 * (src/hip/plan.zig:161-204): stage bit 0 = prepare, bit 1 = GEMV, bit 2 = finish; the workspace carries xq, xs and
 * the planes between calls. */
#define T3_STAGE_PREPARE 1u
#define T3_STAGE_GEMV 2u
#define T3_STAGE_FINISH 4u
int32_t t3_linear_stages(t3_stream stream, const t3_array* x, const t3_array* trellis, const t3_array* suh,
                         const t3_array* svh, t3_decode dec, t3_array* y, void* workspace, size_t workspace_bytes,
                         uint32_t stages);

/* `t3_linear` at its decode rows (1..32) for callers that cannot allocate or pass scratch: code under HIP graph
 * capture, tight serving loops, harnesses that forbid hipMalloc. It has no counterpart in the reference (whose engines
 * own their scratch, src/hip/plan.zig:137-146). The scratch `t3_linear` takes as `workspace` lives in a device array of
 * the library itself, T3_STATIC_SCRATCH_BYTES on every GPU the library runs on, held until the process ends; the call
 * allocates nothing, frees nothing and calls no library routine that could. Same kernels, same launches, same bytes
 * as `t3_linear` for the same operands. Refusals before any launch: more than 32 rows (more than 16 under
 * t3_config.dense_rows_alone = 1, which sends rows 17..32 to the trellis GEMM): T3_Exl3EngineNotImplemented;
 * a call whose scratch (`t3_linear_workspace_bytes`) exceeds T3_STATIC_SCRATCH_BYTES: T3_WorkspaceTooSmall; else as
 * `t3_linear`. All calls on one GPU share that GPU's array: calls that overlap on one GPU (two streams, two threads)
 * race on it; order them on one stream. The first call on a device looks up the array's address there
 * (hipGetSymbolAddress) and clears its counter head on `stream`: make that call outside graph capture. A call that did
 * not run to its end (a failed launch, a reset stream) may leave arrival counters nonzero in the array, which no caller
 * can reach: `t3_linear_static_reset` zeroes the head again with one small fill launch on `stream` (it allocates
 * nothing either), and `t3_linear_static` does the same by itself when one of its own launches reports an error. */
#define T3_STATIC_SCRATCH_BYTES (16u << 20)
int32_t t3_linear_static(t3_stream stream, const t3_array* x, const t3_array* trellis, const t3_array* suh,
                         const t3_array* svh, t3_decode dec, t3_array* y);
int32_t t3_linear_static_reset(t3_stream stream);

/* `t3_linear` plus a bias [out] in x's dtype: one add in x's dtype after the projection's own output rounding, so a
 * sum rounds twice (src/root.zig:358-376 `linearBias`). */
int32_t t3_linear_bias(t3_stream stream, const t3_array* x, const t3_array* trellis, const t3_array* suh,
                       const t3_array* svh, const t3_array* bias, t3_decode dec, t3_array* y, void* workspace,
                       size_t workspace_bytes);

/* How `t3_linear` would run a call, without launching anything: the partition a host or a profiler can read where the
 * reference publishes its launch plans (src/hip/plan.zig:112-204 `dense`). The K slices and tiles a wave depend on the
 * matrix alone, never on the rows of a call: a row's bytes are those of the row alone. Status as `t3_linear`'s checks. */
enum {
    T3_DENSE_ONE_LAUNCH = 0,   /* prepare + GEMV + finish in one kernel */
    T3_DENSE_ARRIVE = 1,       /* prepare launch, then the GEMV whose last workgroup a block runs the finish */
    T3_DENSE_CHAIN = 2,        /* prepare, GEMV, finish */
    T3_DENSE_TRELLIS_GEMM = 3, /* above 32 rows: prepare, the GEMM that decodes in registers, finish */
    T3_DENSE_W_HAT_GEMM = 4    /* from dense_gemm_rows rows: W_hat decode, prepare, plain f16 GEMM, finish */
};
typedef struct t3_linear_plan {
    int32_t path;            /* T3_DENSE_* */
    int32_t launches;
    uint32_t rows, in, out, n;
    uint32_t tiles_a_load;   /* adjacent output tiles one 128-bit load a lane covers (GEMV paths) */
    uint32_t k_slices;       /* planes z [k_slices][rows][out] summed in slice order by the finish */
    uint32_t tiles_a_wave;   /* input tiles a wave walks (GEMV paths; 0 on the GEMM paths) */
    uint32_t workgroups;     /* of the GEMV or GEMM launch */
    uint64_t code_bytes;     /* (in/16)(out/16) n 2: what one call reads of the trellis */
    size_t workspace_bytes;
} t3_linear_plan;
int32_t t3_linear_plan_of(const t3_array* x, const t3_array* trellis, t3_decode dec, t3_linear_plan* plan);

/* W_hat f16 [in, out] from trellis [in/16, out/16, n], bit-exact to format.reconstructInner
 * (src/core/format.zig:276-291; the role of src/core/dense.zig:909-922 `dequantize`). */
int32_t t3_dequant(t3_stream stream, const t3_array* trellis, t3_decode dec, t3_array* w_hat);

/* The resident W_hat (src/core/dense.zig:1323-1345, a host's opt-in: memory for compute): `t3_linear` above
 * t3_config.dense_gemm_rows rows decodes the whole trellis to W_hat on every call; a host that keeps the W_hat of
 * `t3_dequant` calls this instead: prepare, then one plain f16 GEMM that ends with the finish, the same launches on the
 * same operands, so y is `t3_linear`'s W_hat form byte for byte. w_hat F16 [in, out]. Up to 32 rows it refuses with
 * T3_Exl3EngineNotImplemented: decode and verify rows never read a W_hat (dense.zig:1309). Where the GEMM's 256 x 256
 * tiles are few it shares K out over the grid (planes in the workspace, the finish a launch of its own), so a kept W_hat
 * pays at every row count above 32 (measured against `t3_linear` at 4096 -> 14336, us: 64 rows 36 against 41, 512 rows
 * 77 against 103, 2048 rows 235 against 276). `t3_linear_unrot` takes no workspace and so has no K parts:
 * `t3_linear_unrot_parts` is its form for calls of few rows. */
int32_t t3_linear_resident_workspace_bytes(const t3_array* x, const t3_array* w_hat, size_t* bytes);
int32_t t3_linear_resident(t3_stream stream, const t3_array* x, const t3_array* w_hat, const t3_array* suh,
                           const t3_array* svh, t3_array* y, void* workspace, size_t workspace_bytes);

/* The un-rotated weight of a dense linear, made once a weight (src/core/dense.zig:1600-1676 `unrotCols`, `unrotRows`,
 * `unrotWeight`; src/root.zig:392-505 `trunkUnrot` installs it): W_std = act(((H' W_hat H)[i, o] / 128) suh[i] svh[o]),
 * one rounding, written to columns [col0, col0 + out) of w_std [in, N] (F16 or BF16: the activation dtype). A join of up
 * to four linears reading one x is one w_std with the members side by side (dense.zig:1613). Workspace: its head, then
 * six bytes a weight (the W_hat and pass 1's f32 copy), as in the reference. `nonfinite` (device, may be null): a u32 the kernels
 * add the number of weights that left the dtype's range to; the reference keeps such a group on its trellis path
 * (root.zig:456-468). The caller zeroes it before and reads it after the stream has run. */
int32_t t3_unrot_workspace_bytes(const t3_array* trellis, size_t* bytes);
int32_t t3_unrot_weight(t3_stream stream, const t3_array* trellis, const t3_array* suh, const t3_array* svh,
                        t3_decode dec, t3_array* w_std, int64_t col0, uint32_t* nonfinite, void* workspace,
                        size_t workspace_bytes);
/* y [rows, cols] = x [rows, in] W_std[:, col0 : col0 + cols], x, w_std and y in one dtype (F16 or BF16), f32
 * accumulation: one plain GEMM on the matrix cores (w_std's row length a multiple of 8, col0 of 8). Up to 32 rows
 * (src/core/dense.zig:1611 `unrot_min_rows`) it refuses with T3_Exl3EngineNotImplemented: decode and verify rows keep
 * the trellis paths byte for byte. */
int32_t t3_linear_unrot(t3_stream stream, const t3_array* x, const t3_array* w_std, int64_t col0, int64_t cols,
                        t3_array* y);
/* The same product for calls of few rows or a narrow member (no counterpart in the reference, whose W_std product is one
 * MLX matmul whatever the shape): where the GEMM's 256 x 256 tiles are few it shares K out over the grid (f32 planes in
 * the workspace, summed in part order and rounded once by a second launch), so the GPU fills: 4096 -> 14336 at 64 rows
 * 78 -> 29 us. Where the tiles fill the GPU by themselves it is `t3_linear_unrot`'s launch and bytes; with K parts the
 * sums are added in another order and a value can differ from `t3_linear_unrot`'s by a step of the dtype (held to the
 * same bars). Checks and refusals as `t3_linear_unrot`. */
int32_t t3_linear_unrot_workspace_bytes(const t3_array* x, const t3_array* w_std, int64_t col0, int64_t cols, size_t* bytes);
int32_t t3_linear_unrot_parts(t3_stream stream, const t3_array* x, const t3_array* w_std, int64_t col0, int64_t cols,
                              t3_array* y, void* workspace, size_t workspace_bytes);

/* ---- routed experts (src/root.zig:822-904,976-1004) ------------------------------------------------------- */

/* x [B, S, D]; inds (U32/I32) and scores (F32/BF16/F16) [B, S, K], K <= 32; y [B, S, D] in x's dtype.
 * `verify_rows` is accepted and ignored, as in the reference (src/root.zig:822-825). Up to 16 rows: the split-K GEMV
 * chain, two launches (six for large experts at several rows; four or five under decode_form 8 or 3; the same bytes,
 * and t3_moe_plan_of says which). A routed id outside [0, E) is skipped. Gate and up
 * must share a rate (T3_Exl3GateUpRateMismatch); the down's rate may differ (the reference refuses that,
 * src/root.zig:841; this library's kernels take a rate a launch). */
int32_t t3_moe(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
               const t3_array* scores, t3_decode dec, int32_t verify_rows, t3_array* y, void* workspace,
               size_t workspace_bytes);
/* `t3_moe` with the SwiGLU's gate clamped from above and up to [-limit, limit]; limit 1..128 else
 * T3_InvalidExl3Clamp (src/root.zig:1001-1004). */
int32_t t3_moe_clamped(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
                       const t3_array* scores, t3_decode dec, int32_t limit, t3_array* y, void* workspace,
                       size_t workspace_bytes);
/* Where a clamped SwiGLU clamps (src/core/format.zig:80-83 `ClampAt`): gate_in, DeepSeek-V4's and GLM's:
 * silu(min(g, L)) * clamp(u, -L, L); silu_out, Ling-3.1's: min(silu(g), L) * clamp(u, -L, L). */
enum { T3_CLAMP_GATE_IN = 0, T3_CLAMP_SILU_OUT = 1 };
/* `moe`'s chains with the clamp `limit` (0: none; 1..128) at `clamp_at` (src/root.zig:826-833 `moeSwiglu`):
 * `t3_moe` is this at limit 0, `t3_moe_clamped` at gate_in. */
int32_t t3_moe_swiglu(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
                      const t3_array* scores, t3_decode dec, int32_t limit, int32_t clamp_at, t3_array* y,
                      void* workspace, size_t workspace_bytes);
/* `t3_moe` plus an already gated shared-expert output of x's shape and dtype, added at the routed output's
 * rounding point (src/root.zig:976-984). */
int32_t t3_moe_with_shared(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
                           const t3_array* scores, t3_decode dec, int32_t verify_rows, const t3_array* shared,
                           t3_array* y, void* workspace, size_t workspace_bytes);
/* The routed experts with a shared expert inside the same launches: every row also runs each expert of `shared_bank`
 * (same widths and rates as `bank`) at weight 1, summed after the row's routed slots in f32 before the output
 * rounding. limit 0: no clamp; 1..128: `t3_moe_clamped`'s. The role of Qwen3.8's fused shared expert
 * (src/models/qwen38/api.zig:305-312) with the gate left to the caller; the reference's own `moeWithShared` adds a
 * finished tensor instead. */
int32_t t3_moe_shared_expert(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
                             const t3_array* scores, t3_decode dec, int32_t limit, const t3_bank* shared_bank,
                             t3_array* y, void* workspace, size_t workspace_bytes);
/* `t3_moe_shared_expert` (shared_bank NULL: `t3_moe_swiglu` at gate_in; limit 0: no clamp) with a choice of its
 * launches, for profilers and benchmarks that time one stage at a time (the role `t3_linear_stages` has for the dense
 * chain; src/hip/plan.zig:294-364,436-476 publishes the same launches one by one). The workspace carries the stages'
 * results between calls. Up to 16 rows in the two-launch form: bit 0 gate|up + mid, bit 1 down + combine (one to four
 * rows: the mid stage runs inside the down launch, so bit 0 is gate|up alone; the four- and five-launch forms run whole). Above: bit 0 the route, 1 prepare, 2 gate|up GEMM, 3 mid, 4 down GEMM, 5 combine. */
#define T3_MOE_STAGE_GATE_UP 1u
#define T3_MOE_STAGE_DOWN 2u
#define T3_PREFILL_STAGE_ROUTE 1u
#define T3_PREFILL_STAGE_PREPARE 2u
#define T3_PREFILL_STAGE_GEMM_GATE_UP 4u
#define T3_PREFILL_STAGE_MID 8u
#define T3_PREFILL_STAGE_GEMM_DOWN 16u
#define T3_PREFILL_STAGE_COMBINE 32u
int32_t t3_moe_stages(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
                      const t3_array* scores, t3_decode dec, int32_t limit, const t3_bank* shared_bank, t3_array* y,
                      void* workspace, size_t workspace_bytes, uint32_t stages);
/* Decode / verify rows (up to T3_SHARED_ROWS_MAX) of a MoE with a GATED shared expert inside the routed launches
 * (src/models/qwen38/api.zig:305-312 `moeFusedShared`): y = routed + sigmoid(logit) * shared(x), with the roundings of
 * the host's chain it stands for: the routed sum rounds to x's dtype; the shared expert's SwiGLU is the table form in
 * x's dtype (g * sigtab[g]) * u, one rounding an operation (src/models/qwen38/kernels/shared/shared_fin_head_4.metal:1-9);
 * its output rounds to the dtype, is multiplied by sigtab[logit[row]], rounds, and the add rounds (dfin7s.metal:44-50).
 * x F16 or BF16; shared_bank: one expert, the routed bank's widths and rates; sigtab [65536] in x's dtype: the sigmoid
 * of every 16-bit pattern (the host's table); logit [rows] in x's dtype. No clamp. Anything else:
 * T3_Exl3EngineNotImplemented before any launch (the caller keeps its chain). Workspace: t3_moe_workspace_bytes with
 * shared_bank. */
#define T3_SHARED_ROWS_MAX 4 /* src/models/qwen38/shared.zig:346 */
int32_t t3_moe_fused_shared(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds,
                            const t3_array* scores, t3_decode dec, const t3_bank* shared_bank, const t3_array* sigtab,
                            const t3_array* logit, t3_array* y, void* workspace, size_t workspace_bytes);
/* `t3_moe_fused_shared` with the routing inside (src/models/qwen38/api.zig:386-395 `moeFusedSharedRouted`): logits
 * [B, S, E] in x's dtype is the router gemv's output and k the experts a token (1..31, E <= 2048); one more launch
 * in front picks each row's top-k by logit (ties to the lowest id) and their softmax weights renormalised over the k,
 * with the statements of the host's router kernel as the reference restates it (src/models/qwen38/kernels/shared/
 * router_softmax_1..6.metal): the softmax over all experts in f32, each weight rounded to the dtype, their total added
 * up in ascending slot order in the dtype, each weight divided by it. The slots and weights live in the workspace's
 * tail. Exactly one of `logit` and `gate_vec` (else T3_BadExl3Shape, api.zig:399): logit [rows] as `t3_moe_fused_shared`
 * takes it, or gate_vec BF16 [D], the shared gate's weight vector: the router's launch then also takes each row's logit
 * x[row] . gate_vec, in the summation order the reference states for MLX's gemv (src/core/kernels/sources/
 * gate_gemv.metal, gate_sum.metal) and rounded to bf16, at the rows and widths that gemv runs at (x BF16, 2..4 rows,
 * D > 64, D >= 16 rows; else T3_Exl3EngineNotImplemented, api.zig:412-416). */
int32_t t3_moe_fused_shared_routed_workspace_bytes(const t3_array* x, const t3_bank* bank, const t3_array* logits,
                                                   int64_t k, const t3_bank* shared_bank, size_t* bytes);
int32_t t3_moe_fused_shared_routed(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* logits,
                                   int64_t k, t3_decode dec, const t3_bank* shared_bank, const t3_array* sigtab,
                                   const t3_array* logit, const t3_array* gate_vec, t3_array* y, void* workspace,
                                   size_t workspace_bytes);
/* How the routed entry points would run a call, without launching anything (src/hip/plan.zig:283-371 `moe`'s plans):
 * the partitions come from the bank's widths alone. shared_bank may be NULL. Status as `t3_moe`'s checks. */
enum {
    T3_MOE_TWO_LAUNCHES = 0,   /* gate|up + mid, down + combine */
    T3_MOE_FOUR_LAUNCHES = 1,  /* gate|up (prepare inside), mid, down, combine */
    T3_MOE_FIVE_LAUNCHES = 2,  /* prepare, gate|up, mid, down, combine */
    T3_MOE_GROUPED = 4,        /* group, prepare, gate|up, mid, down, combine: the row-slots that read one expert served
                                * together (large experts at two rows or more), the same bytes */
    T3_MOE_PREFILL = 3         /* above 16 rows: route (clear, histogram, scan, place), prepare, gate|up GEMM, mid, down
                                * GEMM, combine */
};
typedef struct t3_moe_plan {
    int32_t path;              /* T3_MOE_* */
    int32_t launches;
    uint32_t rows, row_slots;  /* row_slots = rows (topk + shared slots) */
    uint32_t hidden, inter, topk, shared_slots;
    uint32_t tiles_a_wave_gu, k_slices_gu, tiles_a_load_gu;  /* gate|up GEMV (decode rows) */
    uint32_t tiles_a_wave_dn, k_slices_dn, tiles_a_load_dn;  /* down GEMV */
    uint32_t k_slices_a_workgroup_dn;  /* 2: the two launches' down workgroups hold both K slices (eight waves); same bytes */
    uint32_t item_rows, max_items;                           /* prefill: rows a GEMM item, items at most */
    uint64_t expert_code_bytes;  /* one expert's three matrices */
    size_t workspace_bytes;
    /* prefill: where the route's arrays sit in the workspace (byte offsets; the roles of src/hip/plan.zig:40-45), for a
     * host that reads the routing back: order u32 [row_slots] position -> row-slot; inv u32 [row_slots] row-slot ->
     * position (~0: skipped); items u32 [max_items][4] {expert, first position, rows, 0}; counts u32 [E + S + 2]: rows an
     * expert, then the item count, then the positions placed. 0 on the decode paths. */
    size_t route_order_at, route_inv_at, route_items_at, route_counts_at;
} t3_moe_plan;
int32_t t3_moe_plan_of(const t3_array* x, const t3_bank* bank, const t3_array* inds, const t3_bank* shared_bank,
                       t3_moe_plan* plan);
/* The routed experts under GLM's rounding profile (src/hip/plan.zig:219-247,396-403 `Profile.glm`;
 * src/kernels/hip/decode/decode.hip:8-13): x BF16 times suh in f32 (no f16 rounding of x), the inner products stay f32,
 * gate and up round to bf16 and are limited (limit 0: not), the SiLU rounds to bf16, the product rounds to bf16; y F32
 * [B, S, K, D]: each routed slot's own down finish, no score (the host combines a row's slots and its shared expert). A
 * slot whose id is outside [0, E) is skipped and its output left as it is. Any row count: the decode chain up to 16 rows
 * (the launch forms of t3_moe, the same bytes; MUL1 decoded weight by weight (mul1_defer = 0) and decode_form 8 take the five launches), the
 * prefill chain above. Workspace: t3_moe_workspace_bytes (shared_bank NULL). */
int32_t t3_moe_glm(t3_stream stream, const t3_array* x, const t3_bank* bank, const t3_array* inds, t3_decode dec,
                   int32_t limit, t3_array* y, void* workspace, size_t workspace_bytes);
/* shared_bank: NULL, or the bank `t3_moe_shared_expert` will take (its slots need scratch too). */
int32_t t3_moe_workspace_bytes(const t3_array* x, const t3_bank* bank, const t3_array* inds,
                               const t3_bank* shared_bank, size_t* bytes);

/* ---- pack contract (src/core/spec.zig) ------------------------------------------------------------------- */

#define T3_DECODE_ROWS_MAX 16 /* src/core/spec.zig:59 */
#define T3_REDUCE_MAX_TOPK 32 /* src/core/spec.zig:61 */

/* n halfwords a tile: even, 16..128 (src/core/format.zig:96-100). */
int32_t t3_rate_admitted(int64_t n);
/* T3_Exl3TopKExceedsReduceBank above 32 (src/core/spec.zig:75-77). */
int32_t t3_admit_topk(int64_t topk);
/* A stacked trellis [E, in/16, out/16, n] at or under rate n_max (src/core/spec.zig:80-88): 1 admitted, 0 not. */
int32_t t3_trellis_admitted(const int64_t* shape, int32_t ndim, int64_t experts, int64_t in_dim, int64_t out_dim,
                            int64_t n_max);

/* ---- the quant table (table/config.zig, table/table.zig) -------------------------------------------------------
 * turboexl3 as an mlx-serve quant table: which blocks of a pack's config it claims, what validation names, the bill,
 * the checks a weight passes as it loads, and the table's compute members over loaded weights. JSON arrives as
 * NUL-terminated text. A verdict (`Verdict`, table/table.zig:62,591-593) is its kind plus a reason written to `why`
 * (NUL-terminated, truncated to why_bytes; the reference's error name or message; empty for ok). The plugin kit's ABI
 * struct layouts are not part of the reference tree: these entry points carry the same semantics over this header's own
 * descriptors. */

enum { T3_CLAIM_NO = 0, T3_CLAIM_BY_TYPE = 1, T3_CLAIM_BY_MARKER = 2 };          /* docs/core/glossary.md:220-221 */
enum { T3_VERDICT_OK = 0, T3_VERDICT_UNSUPPORTED = 1, T3_VERDICT_FAILED = 2, T3_VERDICT_TOO_LARGE = 3 };
enum { T3_BLOCK_TRUNK = 0, T3_BLOCK_BANK = 1 };                                    /* table/config.zig:14 */

/* A claimed block (table/config.zig:16-25): a dense trunk's (`trunk_quant`) or a routed bank set's (`expert_quant`). */
typedef struct t3_block {
    int32_t kind;        /* T3_BLOCK_* */
    int32_t codebook;    /* 0 MUL1, 1 MCG */
    int32_t window_bits; /* 8..16 */
    int32_t n;           /* a bank block's rate: halfwords a tile (16 k); 0 for a trunk block */
} t3_block;

/* A loaded weight with its decode (table/table.zig:174-194): `layout` the codebook, `flags` the window's bits, `block`
 * the rate (halfwords a tile). The arrays stay the caller's. */
typedef struct t3_weight {
    t3_array w, scales, biases;
    int32_t layout, flags, block;
} t3_weight;

/* table/config.zig:36-52 `parseBlock`: T3_OK, or NotExl3 / Exl3CodebookUnsupported / Exl3WindowUnsupported /
 * Exl3RateUnsupported. */
int32_t t3_table_parse_block(const char* block_json, t3_block* out);
/* table/config.zig:59-72 `claimFor`: a trunk block always by marker; a bank block by marker on a fully EXL3 Qwen3.8
 * pack, unclamped, where the matrix-engine gate holds (`matrix_gate`: the reference passes MLX's NAX gate; on MI355X
 * the MFMA paths are always there, so a host passes 1). Returns T3_CLAIM_*. */
int32_t t3_table_claims(const char* block_json, const char* config_json, int32_t matrix_gate);
/* table/config.zig:74-85 `validate`: returns T3_VERDICT_*; the reason names an unserved codebook, window, rate, top-k. */
int32_t t3_table_validate(const char* block_json, const char* config_json, char* why, size_t why_bytes);
/* table/config.zig:88-92 `bill`: the weights are the server's loaded arrays, as stored. */
uint64_t t3_table_bill(const char* block_json, const char* model_dir, uint64_t stored);
/* table/table.zig:119-145 `loadTensor`: `<base>.weight` (trellis U16/I16 [in/16, out/16, n]), `.scales` (suh F16 [in]),
 * `.biases` (svh F16 [out]) under a trunk block; in_dim 0 = unchecked. A NULL array is a missing tensor. */
int32_t t3_table_load_tensor(const t3_block* block, const t3_array* weight, const t3_array* scales,
                             const t3_array* biases, uint32_t in_dim, t3_weight* out, char* why, size_t why_bytes);
/* table/table.zig:147-174 `loadBank`: `<base>.{trellis,suh,svh}` under a bank block: trellis U16 [E, in/16, out/16, n]
 * at or under the block's rate, suh F16 [E, in], svh F16 [E, out]. */
int32_t t3_table_load_bank(const t3_block* block, const t3_array* trellis, const t3_array* suh, const t3_array* svh,
                           uint32_t in_dim, t3_weight* out, char* why, size_t why_bytes);
/* table/table.zig:196-201 `matmul`: `t3_linear` with the weight's own decode. */
int32_t t3_table_matmul(t3_stream stream, const t3_weight* w, const t3_array* x, t3_array* y, void* workspace,
                        size_t workspace_bytes, char* why, size_t why_bytes);
int32_t t3_table_matmul_workspace_bytes(const t3_weight* w, const t3_array* x, size_t* bytes);
/* table/table.zig:203-205 `moe`: always refuses: a layer's banks run as one routed SwiGLU. */
int32_t t3_table_moe(char* why, size_t why_bytes);
/* table/table.zig:210-222 `swiglu`: refuses banks that decode differently; limit > 0 runs `t3_moe_clamped`. */
int32_t t3_table_swiglu(t3_stream stream, const t3_weight* gate, const t3_weight* up, const t3_weight* down,
                        const t3_array* x, const t3_array* inds, const t3_array* scores, int32_t limit,
                        int32_t verify_rows, t3_array* y, void* workspace, size_t workspace_bytes, char* why,
                        size_t why_bytes);
int32_t t3_table_swiglu_workspace_bytes(const t3_weight* gate, const t3_weight* up, const t3_weight* down,
                                        const t3_array* x, const t3_array* inds, size_t* bytes);

/* ---- device self-tests (the roles of src/kernels/hip/test/lane.hip) ------------------------------------------ */

/* mcg, mul1, t: device u16 [65536]: every codeword's MCG value, MUL1 value and MUL1 byte sum. */
int32_t t3_test_codebooks(t3_stream stream, uint16_t* mcg, uint16_t* mul1, uint16_t* t);
/* trellis: device u16 [tiles, n]; cw, mcg, mul1: device u16 [tiles, 256] by code position. */
int32_t t3_test_lane(t3_stream stream, const uint16_t* trellis, int64_t n, int32_t window_bits, int64_t tiles,
                     uint16_t* cw, uint16_t* mcg, uint16_t* mul1);
/* in: device f32 [count]; bf16, f16: device u16 [count]: each value narrowed as the kernels narrow an output (nearest even;
 * a NaN stays a quiet NaN: src/test_support.zig:14-19); back: device f32 [count]: the bf16 widened again. */
int32_t t3_test_convert(t3_stream stream, const float* in, uint16_t* bf16, uint16_t* f16, float* back, int64_t count);
/* a f16 [16, 32], b f16 [32, 16] (bits), d f32 [16, 16] = a b through the kernels' MFMA fragments. */
int32_t t3_test_mfma(t3_stream stream, const uint16_t* a, const uint16_t* b, float* d);
/* A measurement, not a test: a plain read of `bytes` device bytes (a multiple of 16, 16-byte aligned), 16 bytes a lane,
 * by `workgroups` workgroups of 256 threads, folded into sink u32 [workgroups * 256]: the read rate the memory system gives
 * a kernel that does nothing else, which the benchmark states beside the 8 TB/s figure (no counterpart in the reference,
 * whose bench quotes the vendor's bandwidth, src/core/bench.zig:217). */
int32_t t3_test_hbm_read(t3_stream stream, const void* src, uint64_t bytes, uint32_t* sink, int32_t workgroups);

#ifdef __cplusplus
}
#endif
#endif
