/*
 * The C ABI called from plain C: no Python, no torch, device memory from hipMalloc, the null stream. Test
 * infrastructure: it links the CPU oracle beside the library and holds the library's outputs to it with the bars of
 * turboexl3 src/hip_tests.zig:326,344,483 (decoded weights to the bit; f32 5e-3, bf16 2.5e-2 of rms).
 *
 *   make -C tests/abi_c && tests/abi_c/abi_check        (on a machine with an MI355X)
 *
 * Exit status 0 and a line a check when everything holds; the first failure prints what differed and exits 1.
 */
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <hip/hip_runtime_api.h>

#include "../../include/turboexl3_hip.h"
#include "../../oracle/t3_oracle.h"

#define HIP_OK(call)                                                                         \
    do {                                                                                     \
        hipError_t e_ = (call);                                                              \
        if (e_ != hipSuccess) {                                                              \
            fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #call, hipGetErrorString(e_)); \
            exit(1);                                                                         \
        }                                                                                    \
    } while (0)

#define T3_DO(call)                                                                          \
    do {                                                                                     \
        int32_t s_ = (call);                                                                 \
        if (s_ != T3_OK) {                                                                   \
            fprintf(stderr, "%s:%d: %s: %s\n", __FILE__, __LINE__, #call, t3_error_name(s_)); \
            exit(1);                                                                         \
        }                                                                                    \
    } while (0)

static uint64_t rng_state = 0x9E3779B97F4A7C15ull;
static uint32_t rnd(void) { /* xorshift64* */
    rng_state ^= rng_state >> 12;
    rng_state ^= rng_state << 25;
    rng_state ^= rng_state >> 27;
    return (uint32_t)((rng_state * 0x2545F4914F6CDD1Dull) >> 32);
}
static float unit(void) { return (float)(rnd() >> 8) / 16777216.0f; }
/* a rough normal: the sum of twelve uniforms less six */
static float normal(void) {
    float s = 0.0f;
    for (int i = 0; i < 12; ++i) s += unit();
    return s - 6.0f;
}

static void* to_device(const void* host, size_t bytes) {
    void* d = NULL;
    HIP_OK(hipMalloc(&d, bytes));
    HIP_OK(hipMemcpy(d, host, bytes, hipMemcpyHostToDevice));
    return d;
}

static t3_array array_of(void* data, int dtype, int ndim, int64_t d0, int64_t d1, int64_t d2, int64_t d3) {
    t3_array a;
    memset(&a, 0, sizeof a);
    a.data = data;
    a.ndim = ndim;
    a.dtype = dtype;
    a.shape[0] = d0;
    a.shape[1] = d1;
    a.shape[2] = d2;
    a.shape[3] = d3;
    return a;
}

typedef struct {
    size_t in_f, out_f, experts;
    uint32_t n;
    uint16_t *trellis, *suh, *svh;       /* host */
    void *d_trellis, *d_suh, *d_svh;     /* device */
} weights;

/* `experts` projections in -> out at n halfwords a tile: uniform codes, scales in [0.5, 1.5), svh / sqrt(in) */
static weights synth(size_t experts, size_t in_f, size_t out_f, uint32_t n) {
    weights w = {in_f, out_f, experts, n, NULL, NULL, NULL, NULL, NULL, NULL};
    const size_t words = experts * (in_f / 16) * (out_f / 16) * n;
    w.trellis = malloc(words * 2);
    w.suh = malloc(experts * in_f * 2);
    w.svh = malloc(experts * out_f * 2);
    for (size_t i = 0; i < words; ++i) w.trellis[i] = (uint16_t)rnd();
    float scale = 1.0f;
    for (size_t v = in_f; v > 1; v >>= 2) scale *= 0.5f; /* 1 / sqrt(in) for in a power of four; near it otherwise */
    for (size_t i = 0; i < experts * in_f; ++i) w.suh[i] = t3o_f32_to_f16((rnd() & 1 ? 1.0f : -1.0f) * (0.5f + unit()));
    for (size_t i = 0; i < experts * out_f; ++i)
        w.svh[i] = t3o_f32_to_f16((rnd() & 1 ? 1.0f : -1.0f) * (0.5f + unit()) * scale);
    w.d_trellis = to_device(w.trellis, words * 2);
    w.d_suh = to_device(w.suh, experts * in_f * 2);
    w.d_svh = to_device(w.svh, experts * out_f * 2);
    return w;
}

static void* workspace = NULL;
static size_t workspace_bytes = 0;
/* the caller's scratch: grown on demand, its head zero-filled once an allocation (the ABI's workspace contract) */
static void reserve(size_t need) {
    if (need <= workspace_bytes) return;
    if (workspace) HIP_OK(hipFree(workspace));
    HIP_OK(hipMalloc(&workspace, need));
    HIP_OK(hipMemset(workspace, 0, T3_WORKSPACE_COUNTER_BYTES));
    workspace_bytes = need;
}

/* x [rows][in] in `dtype` from f32 values; the values the device sees come back in x (rounded to the dtype) */
static void* activations(float* x, size_t count, int dtype) {
    if (dtype == T3_F32) return to_device(x, count * 4);
    uint16_t* h = malloc(count * 2);
    for (size_t i = 0; i < count; ++i) {
        h[i] = dtype == T3_F16 ? t3o_f32_to_f16(x[i]) : t3o_f32_to_bf16(x[i]);
        x[i] = dtype == T3_F16 ? t3o_f16_to_f32(h[i]) : t3o_bf16_to_f32(h[i]);
    }
    void* d = to_device(h, count * 2);
    free(h);
    return d;
}

static void outputs(const void* d_y, float* y, size_t count, int dtype) {
    if (dtype == T3_F32) {
        HIP_OK(hipMemcpy(y, d_y, count * 4, hipMemcpyDeviceToHost));
        return;
    }
    uint16_t* h = malloc(count * 2);
    HIP_OK(hipMemcpy(h, d_y, count * 2, hipMemcpyDeviceToHost));
    for (size_t i = 0; i < count; ++i) y[i] = dtype == T3_F16 ? t3o_f16_to_f32(h[i]) : t3o_bf16_to_f32(h[i]);
    free(h);
}

static int failures = 0;
static void verdict(const char* what, double worst, double bar) {
    printf("%-58s worst %.3e of rms (bar %.1e) %s\n", what, worst, bar, worst <= bar ? "ok" : "FAILED");
    if (!(worst <= bar)) ++failures;
}

static void dense_case(const weights* w, size_t rows, int dtype, int codebook, const char* what) {
    const t3_decode dec = {codebook, 16};
    float* x = malloc(rows * w->in_f * 4);
    for (size_t i = 0; i < rows * w->in_f; ++i) x[i] = normal();
    void* d_x = activations(x, rows * w->in_f, dtype);
    const size_t esz = dtype == T3_F32 ? 4 : 2;
    void* d_y = NULL;
    HIP_OK(hipMalloc(&d_y, rows * w->out_f * esz));
    const t3_array ax = array_of(d_x, dtype, 2, (int64_t)rows, (int64_t)w->in_f, 0, 0);
    const t3_array at = array_of(w->d_trellis, T3_U16, 3, (int64_t)w->in_f / 16, (int64_t)w->out_f / 16, w->n, 0);
    const t3_array asu = array_of(w->d_suh, T3_F16, 1, (int64_t)w->in_f, 0, 0, 0);
    const t3_array asv = array_of(w->d_svh, T3_F16, 1, (int64_t)w->out_f, 0, 0, 0);
    t3_array ay = array_of(d_y, dtype, 2, (int64_t)rows, (int64_t)w->out_f, 0, 0);
    size_t need = 0;
    T3_DO(t3_linear_workspace_bytes(&ax, &at, dec, &need));
    reserve(need);
    T3_DO(t3_linear(NULL, &ax, &at, &asu, &asv, dec, &ay, workspace, workspace_bytes));
    HIP_OK(hipDeviceSynchronize());
    float* y = malloc(rows * w->out_f * 4);
    float* ref = malloc(rows * w->out_f * 4);
    outputs(d_y, y, rows * w->out_f, dtype);
    t3o_project_rows(x, rows, w->trellis, NULL, w->suh, w->svh, w->in_f, w->out_f, w->n, codebook, 0xFFFF, 8, ref);
    double worst = 0.0;
    for (size_t r = 0; r < rows; ++r) {
        const double e = t3o_compare(y + r * w->out_f, ref + r * w->out_f, w->out_f, dtype == T3_F16 ? 0.00048828125 : 0.0);
        if (e > worst) worst = e;
    }
    verdict(what, worst, dtype == T3_BF16 ? 2.5e-2 : 5e-3);
    HIP_OK(hipFree(d_x));
    HIP_OK(hipFree(d_y));
    free(x);
    free(y);
    free(ref);
}

static void dequant_case(const weights* w, int codebook, const char* what) {
    const t3_decode dec = {codebook, 16};
    const size_t count = w->in_f * w->out_f;
    void* d_w = NULL;
    HIP_OK(hipMalloc(&d_w, count * 2));
    const t3_array at = array_of(w->d_trellis, T3_U16, 3, (int64_t)w->in_f / 16, (int64_t)w->out_f / 16, w->n, 0);
    t3_array aw = array_of(d_w, T3_F16, 2, (int64_t)w->in_f, (int64_t)w->out_f, 0, 0);
    T3_DO(t3_dequant(NULL, &at, dec, &aw));
    HIP_OK(hipDeviceSynchronize());
    uint16_t* got = malloc(count * 2);
    uint16_t* want = malloc(count * 2);
    HIP_OK(hipMemcpy(got, d_w, count * 2, hipMemcpyDeviceToHost));
    t3o_reconstruct_inner(w->trellis, w->in_f, w->out_f, w->n, codebook, 0xFFFF, want);
    const int same = memcmp(got, want, count * 2) == 0;
    printf("%-58s %s\n", what, same ? "bit-exact ok" : "FAILED: W_hat differs");
    if (!same) ++failures;
    HIP_OK(hipFree(d_w));
    free(got);
    free(want);
}

static void routed_case(size_t rows, const char* what) {
    const size_t experts = 6, hidden = 512, inter = 256, topk = 3;
    const uint32_t n = 48;
    const int limit = 7;
    const t3_decode dec = {T3O_MCG, 16};
    const weights g = synth(experts, hidden, inter, n), u = synth(experts, hidden, inter, n),
                  d = synth(experts, inter, hidden, n);
    float* x = malloc(rows * hidden * 4);
    for (size_t i = 0; i < rows * hidden; ++i) x[i] = normal();
    void* d_x = activations(x, rows * hidden, T3_F32);
    int32_t* slots = malloc(rows * topk * 4);
    float* scores = malloc(rows * topk * 4);
    for (size_t r = 0; r < rows; ++r)
        for (size_t k = 0; k < topk; ++k) {
            slots[r * topk + k] = (int32_t)((r + 2 * k) % experts);  /* distinct within a row */
            scores[r * topk + k] = 0.1f + 0.3f * unit();
        }
    slots[topk - 1] = (int32_t)experts + 3;  /* one id outside the bank: skipped, as the reference skips it */
    void* d_slots = to_device(slots, rows * topk * 4);
    void* d_scores = to_device(scores, rows * topk * 4);
    void* d_y = NULL;
    HIP_OK(hipMalloc(&d_y, rows * hidden * 4));
    const t3_array ax = array_of(d_x, T3_F32, 3, 1, (int64_t)rows, (int64_t)hidden, 0);
    const t3_array ai = array_of(d_slots, T3_I32, 3, 1, (int64_t)rows, (int64_t)topk, 0);
    const t3_array as = array_of(d_scores, T3_F32, 3, 1, (int64_t)rows, (int64_t)topk, 0);
    t3_array ay = array_of(d_y, T3_F32, 3, 1, (int64_t)rows, (int64_t)hidden, 0);
    t3_bank bank;
    const weights* p[3] = {&g, &u, &d};
    t3_proj* q[3] = {&bank.gate, &bank.up, &bank.down};
    for (int i = 0; i < 3; ++i) {
        q[i]->trellis = array_of(p[i]->d_trellis, T3_U16, 4, (int64_t)experts, (int64_t)p[i]->in_f / 16,
                                 (int64_t)p[i]->out_f / 16, n);
        q[i]->suh = array_of(p[i]->d_suh, T3_F16, 2, (int64_t)experts, (int64_t)p[i]->in_f, 0, 0);
        q[i]->svh = array_of(p[i]->d_svh, T3_F16, 2, (int64_t)experts, (int64_t)p[i]->out_f, 0, 0);
    }
    size_t need = 0;
    T3_DO(t3_moe_workspace_bytes(&ax, &bank, &ai, NULL, &need));
    reserve(need);
    T3_DO(t3_moe_clamped(NULL, &ax, &bank, &ai, &as, dec, limit, &ay, workspace, workspace_bytes));
    HIP_OK(hipDeviceSynchronize());
    float* y = malloc(rows * hidden * 4);
    float* ref = malloc(hidden * 4);
    outputs(d_y, y, rows * hidden, T3_F32);
    const t3o_bank ob = {experts, hidden, inter, n, n, g.trellis, g.suh, g.svh, u.trellis, u.suh, u.svh,
                         d.trellis, d.suh, d.svh};
    double worst = 0.0;
    for (size_t r = 0; r < rows; ++r) {
        t3o_moe_row_clamped_at(&ob, T3O_MCG, 0xFFFF, (float)limit, T3O_CLAMP_GATE_IN, x + r * hidden, slots + r * topk,
                               scores + r * topk, topk, ref, NULL);
        const double e = t3o_compare(y + r * hidden, ref, hidden, 0.0);
        if (e > worst) worst = e;
    }
    verdict(what, worst, 5e-3);
}

/* a refusal names itself before anything is launched and leaves y as it was (docs/core/api.md:10-12) */
static void refusal_case(const weights* w) {
    float x[96] = {0};
    void* d_x = to_device(x, sizeof x);
    float fill[4] = {7.0f, 7.0f, 7.0f, 7.0f};
    void* d_y = to_device(fill, sizeof fill);
    const t3_decode dec = {T3O_MCG, 16};
    const t3_array ax = array_of(d_x, T3_F32, 2, 1, 96, 0, 0);  /* 96 inputs: not the trellis's width */
    const t3_array at = array_of(w->d_trellis, T3_U16, 3, (int64_t)w->in_f / 16, (int64_t)w->out_f / 16, w->n, 0);
    const t3_array asu = array_of(w->d_suh, T3_F16, 1, (int64_t)w->in_f, 0, 0, 0);
    const t3_array asv = array_of(w->d_svh, T3_F16, 1, (int64_t)w->out_f, 0, 0, 0);
    t3_array ay = array_of(d_y, T3_F32, 2, 1, (int64_t)w->out_f, 0, 0);
    const int32_t st = t3_linear(NULL, &ax, &at, &asu, &asv, dec, &ay, workspace, workspace_bytes);
    HIP_OK(hipDeviceSynchronize());
    float back[4];
    HIP_OK(hipMemcpy(back, d_y, sizeof back, hipMemcpyDeviceToHost));
    const int ok = st == T3_BadExl3Shape && memcmp(back, fill, sizeof fill) == 0;
    printf("%-58s %s (%s)\n", "a call with the wrong width is refused, y untouched", ok ? "ok" : "FAILED", t3_error_name(st));
    if (!ok) ++failures;
}

int main(void) {
    int count = 0;
    if (hipGetDeviceCount(&count) != hipSuccess || count < 1) {
        fprintf(stderr, "abi_check: no HIP device\n");
        return 2;
    }
    HIP_OK(hipSetDevice(0));
    const weights w = synth(1, 1024, 512, 64);
    dequant_case(&w, T3O_MCG, "t3_dequant 1024 x 512 K4 MCG");
    dequant_case(&w, T3O_MUL1, "t3_dequant 1024 x 512 K4 MUL1");
    dense_case(&w, 1, T3_F16, T3O_MCG, "t3_linear 1 row f16 MCG (one launch)");
    dense_case(&w, 5, T3_F32, T3O_MUL1, "t3_linear 5 rows f32 MUL1 (chain)");
    dense_case(&w, 32, T3_BF16, T3O_MCG, "t3_linear 32 rows bf16 MCG");
    dense_case(&w, 40, T3_BF16, T3O_MCG, "t3_linear 40 rows bf16 MCG (trellis GEMM)");
    routed_case(2, "t3_moe_clamped 2 rows top-3 of 6, one id skipped, f32");
    routed_case(20, "t3_moe_clamped 20 rows (prefill chain), f32");
    refusal_case(&w);
    /* the contract's other half: every call left the workspace's head zero */
    unsigned char* head = malloc(T3_WORKSPACE_COUNTER_BYTES);
    HIP_OK(hipMemcpy(head, workspace, T3_WORKSPACE_COUNTER_BYTES, hipMemcpyDeviceToHost));
    int zero = 1;
    for (size_t i = 0; i < T3_WORKSPACE_COUNTER_BYTES; ++i) zero &= head[i] == 0;
    printf("%-58s %s\n", "the workspace's counter head is zero after every call", zero ? "ok" : "FAILED");
    if (!zero) ++failures;
    printf(failures ? "abi_check: %d check(s) FAILED\n" : "abi_check: all checks hold\n", failures);
    return failures ? 1 : 0;
}
