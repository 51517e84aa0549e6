/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE.
 *
 * A CPU restatement, in plain C, of the turboexl3 host reference for the EXL3 projection path. Only tests,
 * the smoke check and the benchmark's cpu_baseline leg may link or call it; the HIP library never does.
 *
 * Each function names the reference lines it follows (paths relative to the turboexl3 source tree).
 * Arithmetic rules kept from the reference: strict f32 (no contraction; build with -ffp-contract=off), one
 * fused multiply-add (the MUL1 map), f32 -> f16 round-to-nearest-even, H128 as the dense signed sum with the
 * scale folded into every entry.
 *
 * How each part is pinned (see tests/test_oracle_pins.py):
 *   codebooks        known answers (src/core/format.zig:427-431,441-445), byte-sum identity, exhaustive
 *                    cross-check of two independent formulations
 *   unpack / lanes   bit-by-bit definition vs funnel reader vs 4-word lane plan at every even n; packer round trip
 *   perm             permutation property + perm[0], perm[1], perm[4]
 *   hadamard128      involution, Sylvester sign rule, butterfly equivalence
 *   project          128x128 K4 vs reconstruct_public matvec within 2 % of max (src/core/format.zig:534-571)
 *   moe_row          slot order = summation order; clamp rule including NaN pass-through
 * The exact f32 output bits of hadamard128 / project / moe_row have no golden vectors in the reference (its
 * tests recompute them at run time), so those are pinned by source-following plus the invariants above:
 * "parity unpinned" at the bit level, tolerance-pinned otherwise.
 */
#ifndef T3_ORACLE_H
#define T3_ORACLE_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { T3O_MUL1 = 0, T3O_MCG = 1 };
enum { T3O_CLAMP_GATE_IN = 0, T3O_CLAMP_SILU_OUT = 1 };

/* f16 <-> f32 (src/core/format.zig:140-146) */
float t3o_f16_to_f32(uint16_t bits);
uint16_t t3o_f32_to_f16(float v);
/* bf16 round-to-nearest-even with quiet NaN (src/kernels/hip/common.hpp:24-29) */
uint16_t t3o_f32_to_bf16(float v);
float t3o_bf16_to_f32(uint16_t bits);

/* codebooks (src/core/format.zig:149-174) */
uint16_t t3o_decode_mcg(uint16_t cw);
uint16_t t3o_decode_mul1(uint16_t cw);
uint32_t t3o_mul1_bytesum(uint16_t cw);
uint16_t t3o_decode_codeword(uint16_t cw, int codebook);

/* rate helpers (src/core/format.zig:87-133): n halfwords a tile, even, 16..128 */
int t3o_rate_ok(uint64_t n);
uint32_t t3o_bit_end(uint32_t n, uint32_t t);
/* window mask for w in 8..16 (src/core/format.zig:41-69); 0 if not admitted */
uint32_t t3o_window_mask(int bits);

/* tile readers: three independent formulations of the same 256 codewords */
void t3o_unpack_tile(const uint16_t* words, uint32_t n, uint16_t out[256]);           /* format.zig:182-200 */
uint16_t t3o_codeword_by_definition(const uint16_t* words, uint32_t n, uint32_t t);   /* format.zig:202-222 */
void t3o_lane_codewords(const uint16_t* words, uint32_t n, uint32_t lane, uint16_t out[8]); /* lane.zig:32-73 */

/* packer for tests (src/core/format.zig:395-423): 256 K-bit symbols -> n = 16 K halfwords */
void t3o_pack_symbols(const uint16_t* symbols, uint32_t k, uint16_t* out);

/* code position -> row-major tile index (src/core/format.zig:237-256) */
void t3o_tensor_core_perm(uint32_t out[256]);

/* one tile's 256 weights, f16 bits, row-major [16][16] (src/core/format.zig:225-234) */
void t3o_decode_tile(const uint16_t* words, uint32_t n, int codebook, uint32_t mask, uint16_t out[256]);

/* W_hat [in, out] f16 bits from trellis [in/16, out/16, n] (src/core/format.zig:276-291) */
void t3o_reconstruct_inner(const uint16_t* trellis, size_t in_f, size_t out_f, uint32_t n, int codebook,
                           uint32_t mask, uint16_t* out);
/* W_std = diag(suh) H W_hat H diag(svh), f16 bits (src/core/format.zig:295-331) */
int t3o_reconstruct_public(const uint16_t* trellis, const uint16_t* suh, const uint16_t* svh, size_t in_f,
                           size_t out_f, uint32_t n, int codebook, uint32_t mask, uint16_t* out);

/* H128, natural order, scaled 1/sqrt(128), in place (src/core/format.zig:258-273) */
void t3o_hadamard128(float v[128]);

/* the three stages of a projection and the whole (src/core/format.zig:334-389) */
void t3o_prepare_input(const float* x, const uint16_t* suh, size_t in_f, float* out);
void t3o_inner_gemv(const uint16_t* trellis, const float* transformed, size_t in_f, size_t out_f, uint32_t n,
                    int codebook, uint32_t mask, float* out);
void t3o_finish_output(const float* inner, const uint16_t* svh, size_t out_f, float* out);
void t3o_project(const float* x, const uint16_t* trellis, const uint16_t* suh, const uint16_t* svh, size_t in_f,
                 size_t out_f, uint32_t n, int codebook, uint32_t mask, float* y);

/* `rows` rows through one projection on a W_hat decoded once (src/core/ref.zig:241-260): the bits of
 * t3o_project per row; `threads` > 1 splits output columns over OpenMP threads without changing any sum's order.
 * w_hat may be NULL (decoded internally). */
int t3o_project_rows(const float* x, size_t rows, const uint16_t* trellis, const uint16_t* w_hat,
                     const uint16_t* suh, const uint16_t* svh, size_t in_f, size_t out_f, uint32_t n, int codebook,
                     uint32_t mask, int threads, float* y);

/* SwiGLU element rules (src/core/ref.zig:119-140) */
float t3o_swiglu_clamped(float g, float u, float limit);
float t3o_swiglu_clamped_out(float g, float u, float limit);

/* A bank: expert e on axis 0 (src/core/ref.zig:9-43). gate/up: hidden -> inter at n_gu; down: inter -> hidden
 * at n_dn (the reference holds one rate; per-projection rates are this build's extension for mixed packs). */
typedef struct {
    size_t experts, hidden, inter;
    uint32_t n_gu, n_dn;
    const uint16_t *gate_t, *gate_suh, *gate_svh;
    const uint16_t *up_t, *up_suh, *up_svh;
    const uint16_t *down_t, *down_suh, *down_svh;
} t3o_bank;

/* one row over its slots in slot order (src/core/ref.zig:154-190). hits[3] = {gate, up, total} may be NULL.
 * slots outside [0, experts) are skipped. */
int t3o_moe_row_clamped_at(const t3o_bank* b, int codebook, uint32_t mask, float limit, int clamp_at,
                           const float* x, const int32_t* slots, const float* scores, size_t topk, float* y,
                           size_t hits[3]);

/* max |got - ref| / rms(ref) (src/core/ref.zig:193-204); half_ulp > 0 discounts the store rounding (:206-218) */
double t3o_compare(const float* got, const float* ref, size_t len, double half_ulp);

/* partition pins restated from src/hip/plan.zig:86-109,249-260 (the reference's launch plan; test pins only) */
uint32_t t3o_rb_cap(uint32_t rows, uint32_t cap);
uint32_t t3o_bt_for(uint32_t rb);
uint32_t t3o_ks_for(uint32_t in_f, uint32_t out_f);
uint32_t t3o_ks_gu(uint32_t hidden, uint32_t ks_max);
uint32_t t3o_ks_dn(uint32_t inter, uint32_t ks_max);

#ifdef __cplusplus
}
#endif
#endif
