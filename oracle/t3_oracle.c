/*
 * TEST INFRASTRUCTURE, NOT PRODUCT CODE: the CPU restatement of the turboexl3 host reference (see t3_oracle.h).
 * Build: gcc -O2 -std=c11 -ffp-contract=off -fno-fast-math -fopenmp -fPIC -shared (oracle/Makefile).
 */
#include "t3_oracle.h"

#include <math.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define TILE 16u
#define TILE_VALUES 256u
#define HAD 128u

static const float kHadScale = 0.08838834764831845f; /* src/core/format.zig:14 */

/* ---- scalar conversions ------------------------------------------------------------------------------- */

static inline uint32_t f32_bits(float v) {
    uint32_t u;
    memcpy(&u, &v, 4);
    return u;
}
static inline float bits_f32(uint32_t u) {
    float v;
    memcpy(&v, &u, 4);
    return v;
}

float t3o_f16_to_f32(uint16_t h) {
    const uint32_t sign = (uint32_t)(h & 0x8000u) << 16;
    const uint32_t exp = (h >> 10) & 0x1Fu;
    uint32_t man = h & 0x3FFu;
    if (exp == 0x1Fu) return bits_f32(sign | 0x7F800000u | (man << 13));
    if (exp != 0) return bits_f32(sign | ((exp + 112u) << 23) | (man << 13));
    if (man == 0) return bits_f32(sign);
    /* subnormal: value = man * 2^-24 */
    int e = -1;
    do {
        man <<= 1;
        ++e;
    } while (!(man & 0x400u));
    return bits_f32(sign | ((uint32_t)(112 - e) << 23) | ((man & 0x3FFu) << 13));
}

/* round-to-nearest-even, overflow to infinity, NaN kept quiet */
uint16_t t3o_f32_to_f16(float v) {
    const uint32_t u = f32_bits(v);
    const uint16_t sign = (uint16_t)((u >> 16) & 0x8000u);
    const uint32_t a = u & 0x7FFFFFFFu;
    if (a >= 0x7F800000u) return (uint16_t)(sign | (a > 0x7F800000u ? 0x7E00u | ((a >> 13) & 0x3FFu) : 0x7C00u));
    if (a >= 0x477FF000u) return (uint16_t)(sign | 0x7C00u); /* >= 65520 rounds to inf */
    if (a >= 0x38800000u) {                                    /* normal f16 range */
        const uint32_t r = a - 0x38000000u;                    /* rebias 127 -> 15 */
        uint32_t h = r >> 13;
        const uint32_t rem = r & 0x1FFFu;
        if (rem > 0x1000u || (rem == 0x1000u && (h & 1u))) ++h; /* may carry into the exponent: still right */
        return (uint16_t)(sign | h);
    }
    if (a < 0x33000000u) return sign; /* below half the smallest subnormal (2^-25) rounds to zero; ties handled below */
    /* subnormal result: man24 * 2^(e-150) -> units of 2^-24 */
    const int e = (int)(a >> 23);
    const uint32_t man = (a & 0x7FFFFFu) | 0x800000u;
    const int shift = 126 - e; /* e in [102, 112] -> shift in [14, 24] */
    uint32_t h = man >> shift;
    const uint32_t rem = man & ((1u << shift) - 1u);
    const uint32_t half = 1u << (shift - 1);
    if (rem > half || (rem == half && (h & 1u))) ++h;
    return (uint16_t)(sign | h);
}

uint16_t t3o_f32_to_bf16(float v) {
    uint32_t u = f32_bits(v);
    if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7FFFu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
float t3o_bf16_to_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }

static inline float round_half(float v) { return t3o_f16_to_f32(t3o_f32_to_f16(v)); }

/* ---- codebooks (src/core/format.zig:149-174) ------------------------------------------------------------- */

uint16_t t3o_decode_mcg(uint16_t cw) {
    const uint32_t mixed = (uint32_t)cw * 0xCBAC1FEDu;
    const uint32_t pair = 0x3B603B60u ^ (mixed & 0x8FFF8FFFu);
    const float lo = t3o_f16_to_f32((uint16_t)(pair & 0xFFFFu));
    const float hi = t3o_f16_to_f32((uint16_t)(pair >> 16));
    return t3o_f32_to_f16(lo + hi);
}

uint32_t t3o_mul1_bytesum(uint16_t cw) {
    const uint32_t mixed = (uint32_t)cw * 0x83DCD12Du;
    return (mixed & 0xFFu) + ((mixed >> 8) & 0xFFu) + ((mixed >> 16) & 0xFFu) + (mixed >> 24);
}

uint16_t t3o_decode_mul1(uint16_t cw) {
    const float h = t3o_f16_to_f32((uint16_t)(0x6400u + t3o_mul1_bytesum(cw)));
    return t3o_f32_to_f16(fmaf(h, t3o_f16_to_f32(0x1EEEu), t3o_f16_to_f32(0xC931u)));
}

uint16_t t3o_decode_codeword(uint16_t cw, int codebook) {
    return codebook == T3O_MCG ? t3o_decode_mcg(cw) : t3o_decode_mul1(cw);
}

/* ---- rates and windows ------------------------------------------------------------------------------- */

int t3o_rate_ok(uint64_t n) { return n % 2 == 0 && n >= 16 && n <= 128; }
uint32_t t3o_bit_end(uint32_t n, uint32_t t) { return ((t + 1u) * n) >> 4; }
uint32_t t3o_window_mask(int bits) {
    if (bits < 8 || bits > 16) return 0;
    return (1u << bits) - 1u;
}

/* ---- tile readers ------------------------------------------------------------------------------------ */

static inline uint32_t word_at(const uint16_t* words, uint32_t index) {
    return (uint32_t)words[2u * index] | ((uint32_t)words[2u * index + 1u] << 16);
}

/* pairs of weights through one 64-bit funnel (src/core/format.zig:182-200) */
void t3o_unpack_tile(const uint16_t* words, uint32_t n, uint16_t out[256]) {
    const uint32_t word_count = n / 2u, total = TILE * n;
    for (uint32_t pair = 0; pair < 128u; ++pair) {
        const uint32_t e0 = t3o_bit_end(n, 2u * pair), e1 = t3o_bit_end(n, 2u * pair + 1u);
        const uint32_t first_bit = e0 + total - 16u; /* window 2*pair starts here */
        const uint32_t end_bit = e1 + total;         /* window 2*pair+1 ends here (exclusive) */
        const uint32_t i_hi = first_bit / 32u, i_lo = (end_bit - 1u) / 32u;
        const uint32_t shift = (i_lo + 1u) * 32u - end_bit;
        const uint64_t merged = ((uint64_t)word_at(words, i_hi % word_count) << 32) | word_at(words, i_lo % word_count);
        const uint32_t funnel = (uint32_t)(merged >> shift);
        const uint32_t fresh = e1 - e0;
        out[2u * pair] = (uint16_t)((funnel >> fresh) & 0xFFFFu);
        out[2u * pair + 1u] = (uint16_t)(funnel & 0xFFFFu);
    }
}

/* the plain definition: 16 stream bits, MSB first, ending at bit_end(t), circular (format.zig:202-222) */
uint16_t t3o_codeword_by_definition(const uint16_t* words, uint32_t n, uint32_t t) {
    const uint32_t total = TILE * n, end = t3o_bit_end(n, t);
    uint32_t cw = 0;
    for (uint32_t i = 0; i < 16u; ++i) {
        const uint32_t j = (end + total - 16u + i) % total;
        const uint32_t w = word_at(words, j / 32u);
        cw = (cw << 1) | ((w >> (31u - (j % 32u))) & 1u);
    }
    return (uint16_t)cw;
}

/* lane plan: four words from `base`, each window a (word, shift) pair (src/core/lane.zig:32-73) */
void t3o_lane_codewords(const uint16_t* words, uint32_t n, uint32_t lane, uint16_t out[8]) {
    const uint32_t nw = n / 2u;
    const uint32_t base = ((((8u * lane + 1u) * n) >> 4) + 16u * n - 16u) >> 5;
    uint32_t w[4];
    for (uint32_t i = 0; i < 4u; ++i) w[i] = word_at(words, (base + i) % nw);
    const uint32_t wprev = word_at(words, (base + nw - 1u) % nw);
    for (uint32_t m = 0; m < 8u; ++m) {
        const uint32_t off = (((8u * lane + m + 1u) * n) >> 4) + 16u * n - 32u * base;
        const uint32_t q = (off - 1u) >> 5, sh = 32u * (q + 1u) - off;
        const uint32_t hi = w[q], lo = q == 0 ? wprev : w[q - 1u];
        const uint32_t v = sh == 0 ? hi : ((hi >> sh) | (lo << (32u - sh)));
        out[m] = (uint16_t)(v & 0xFFFFu);
    }
}

/* exllamav3 pack.cu as the reference restates it (src/core/format.zig:395-423) */
void t3o_pack_symbols(const uint16_t* symbols, uint32_t k, uint16_t* out) {
    uint16_t emitted[256];
    const uint32_t kmask = (1u << k) - 1u;
    uint32_t i = 0, j = 0;
    for (uint32_t row = 0; row < 16u; ++row) {
        uint32_t buf = 0;
        int room = 32;
        for (uint32_t col = 0; col < 16u; ++col, ++i) {
            room -= (int)k;
            buf |= ((uint32_t)symbols[i] & kmask) << room;
            if (room <= 16) {
                emitted[j++] = (uint16_t)(buf >> 16);
                buf <<= 16;
                room += 16;
            }
        }
    }
    const uint32_t halfwords = TILE_VALUES * k / 16u;
    for (uint32_t w = 0; w < halfwords / 2u; ++w) { /* SWAP16 inside each uint32 */
        out[2u * w] = emitted[2u * w + 1u];
        out[2u * w + 1u] = emitted[2u * w];
    }
}

void t3o_tensor_core_perm(uint32_t out[256]) {
    static const uint32_t row_add[4] = {0u, 1u, 8u, 9u};
    for (uint32_t p = 0; p < 256u; ++p) {
        const uint32_t thr = p / 8u, i = p % 8u;
        const uint32_t row = 2u * (thr % 4u) + row_add[i % 4u];
        const uint32_t col = thr / 4u + 8u * (i / 4u);
        out[p] = row * 16u + col;
    }
}

void t3o_decode_tile(const uint16_t* words, uint32_t n, int codebook, uint32_t mask, uint16_t out[256]) {
    uint16_t cw[256];
    uint32_t perm[256];
    t3o_unpack_tile(words, n, cw);
    t3o_tensor_core_perm(perm);
    for (uint32_t p = 0; p < 256u; ++p) out[perm[p]] = t3o_decode_codeword((uint16_t)(cw[p] & mask), codebook);
}

void t3o_reconstruct_inner(const uint16_t* trellis, size_t in_f, size_t out_f, uint32_t n, int codebook,
                           uint32_t mask, uint16_t* out) {
    const size_t in_tiles = in_f / TILE, out_tiles = out_f / TILE;
#pragma omp parallel for schedule(static)
    for (size_t tk = 0; tk < in_tiles; ++tk) {
        uint16_t tile[256];
        for (size_t tn = 0; tn < out_tiles; ++tn) {
            t3o_decode_tile(trellis + (tk * out_tiles + tn) * n, n, codebook, mask, tile);
            for (size_t r = 0; r < TILE; ++r)
                memcpy(out + (tk * TILE + r) * out_f + tn * TILE, tile + r * TILE, TILE * sizeof(uint16_t));
        }
    }
}

/* ---- Hadamard and the projection stages ------------------------------------------------------------------ */

void t3o_hadamard128(float v[128]) {
    float tmp[128];
    for (uint32_t r = 0; r < HAD; ++r) {
        float acc = 0.0f;
        for (uint32_t k = 0; k < HAD; ++k) {
            const float entry = (__builtin_popcount(r & k) & 1) ? -kHadScale : kHadScale;
            acc += entry * v[k];
        }
        tmp[r] = acc;
    }
    memcpy(v, tmp, sizeof tmp);
}

void t3o_prepare_input(const float* x, const uint16_t* suh, size_t in_f, float* out) {
    for (size_t i = 0; i < in_f; ++i) out[i] = round_half(x[i]) * t3o_f16_to_f32(suh[i]);
    for (size_t b = 0; b < in_f; b += HAD) {
        t3o_hadamard128(out + b);
        for (size_t i = 0; i < HAD; ++i) out[b + i] = round_half(out[b + i]);
    }
}

void t3o_inner_gemv(const uint16_t* trellis, const float* transformed, size_t in_f, size_t out_f, uint32_t n,
                    int codebook, uint32_t mask, float* out) {
    const size_t in_tiles = in_f / TILE, out_tiles = out_f / TILE;
    uint16_t tile[256];
    memset(out, 0, out_f * sizeof(float));
    for (size_t tk = 0; tk < in_tiles; ++tk)
        for (size_t tn = 0; tn < out_tiles; ++tn) {
            t3o_decode_tile(trellis + (tk * out_tiles + tn) * n, n, codebook, mask, tile);
            for (size_t r = 0; r < TILE; ++r) {
                const float xv = transformed[tk * TILE + r];
                for (size_t c = 0; c < TILE; ++c) out[tn * TILE + c] += xv * t3o_f16_to_f32(tile[r * TILE + c]);
            }
        }
    for (size_t i = 0; i < out_f; ++i) out[i] = round_half(out[i]);
}

void t3o_finish_output(const float* inner, const uint16_t* svh, size_t out_f, float* out) {
    memcpy(out, inner, out_f * sizeof(float));
    for (size_t b = 0; b < out_f; b += HAD) t3o_hadamard128(out + b);
    for (size_t i = 0; i < out_f; ++i) out[i] = round_half(out[i] * t3o_f16_to_f32(svh[i]));
}

void t3o_project(const float* x, const uint16_t* trellis, const uint16_t* suh, const uint16_t* svh, size_t in_f,
                 size_t out_f, uint32_t n, int codebook, uint32_t mask, float* y) {
    float* transformed = (float*)malloc(in_f * sizeof(float));
    float* inner = (float*)malloc(out_f * sizeof(float));
    t3o_prepare_input(x, suh, in_f, transformed);
    t3o_inner_gemv(trellis, transformed, in_f, out_f, n, codebook, mask, inner);
    t3o_finish_output(inner, svh, out_f, y);
    free(transformed);
    free(inner);
}

int t3o_project_rows(const float* x, size_t rows, const uint16_t* trellis, const uint16_t* w_hat,
                     const uint16_t* suh, const uint16_t* svh, size_t in_f, size_t out_f, uint32_t n, int codebook,
                     uint32_t mask, int threads, float* y) {
    uint16_t* owned = NULL;
    if (!w_hat) {
        owned = (uint16_t*)malloc(in_f * out_f * sizeof(uint16_t));
        if (!owned) return -1;
        t3o_reconstruct_inner(trellis, in_f, out_f, n, codebook, mask, owned);
        w_hat = owned;
    }
    float* transformed = (float*)malloc(rows * in_f * sizeof(float));
    float* inner = (float*)malloc(rows * out_f * sizeof(float));
    if (!transformed || !inner) {
        free(owned);
        free(transformed);
        free(inner);
        return -1;
    }
    for (size_t r = 0; r < rows; ++r) t3o_prepare_input(x + r * in_f, suh, in_f, transformed + r * in_f);
    /* each output column's sum runs k ascending, as t3o_inner_gemv's does; columns are independent */
    const size_t blocks = out_f / HAD;
    (void)threads;
#pragma omp parallel for schedule(static) num_threads(threads > 0 ? threads : 1)
    for (size_t b = 0; b < blocks; ++b) {
        float wrow[HAD];
        for (size_t r = 0; r < rows; ++r) {
            float acc[HAD];
            memset(acc, 0, sizeof acc);
            const float* tr = transformed + r * in_f;
            for (size_t k = 0; k < in_f; ++k) {
                const uint16_t* wk = w_hat + k * out_f + b * HAD;
                const float xv = tr[k];
                for (size_t c = 0; c < HAD; ++c) wrow[c] = t3o_f16_to_f32(wk[c]);
                for (size_t c = 0; c < HAD; ++c) acc[c] += xv * wrow[c];
            }
            for (size_t c = 0; c < HAD; ++c) inner[r * out_f + b * HAD + c] = round_half(acc[c]);
        }
    }
    for (size_t r = 0; r < rows; ++r) t3o_finish_output(inner + r * out_f, svh, out_f, y + r * out_f);
    free(owned);
    free(transformed);
    free(inner);
    return 0;
}

int t3o_reconstruct_public(const uint16_t* trellis, const uint16_t* suh, const uint16_t* svh, size_t in_f,
                           size_t out_f, uint32_t n, int codebook, uint32_t mask, uint16_t* out) {
    uint16_t* inner = (uint16_t*)malloc(in_f * out_f * sizeof(uint16_t));
    float* w = (float*)malloc(in_f * out_f * sizeof(float));
    if (!inner || !w) {
        free(inner);
        free(w);
        return -1;
    }
    t3o_reconstruct_inner(trellis, in_f, out_f, n, codebook, mask, inner);
    for (size_t i = 0; i < in_f * out_f; ++i) w[i] = t3o_f16_to_f32(inner[i]);
    float vec[128];
    for (size_t rb = 0; rb < in_f; rb += HAD) /* H over input blocks, column by column */
        for (size_t c = 0; c < out_f; ++c) {
            for (size_t r = 0; r < HAD; ++r) vec[r] = w[(rb + r) * out_f + c];
            t3o_hadamard128(vec);
            for (size_t r = 0; r < HAD; ++r) w[(rb + r) * out_f + c] = vec[r];
        }
    for (size_t r = 0; r < in_f; ++r) {
        const float s = t3o_f16_to_f32(suh[r]);
        for (size_t c = 0; c < out_f; ++c) w[r * out_f + c] *= s;
    }
    for (size_t cb = 0; cb < out_f; cb += HAD) /* H over output blocks, row by row */
        for (size_t r = 0; r < in_f; ++r) t3o_hadamard128(w + r * out_f + cb);
    for (size_t c = 0; c < out_f; ++c) {
        const float s = t3o_f16_to_f32(svh[c]);
        for (size_t r = 0; r < in_f; ++r) w[r * out_f + c] *= s;
    }
    for (size_t i = 0; i < in_f * out_f; ++i) out[i] = t3o_f32_to_f16(w[i]);
    free(inner);
    free(w);
    return 0;
}

/* ---- routed experts (src/core/ref.zig) --------------------------------------------------------------- */

float t3o_swiglu_clamped(float g, float u, float limit) {
    float gc = g, uc = u;
    if (limit > 0.0f) {
        gc = g > limit ? limit : g; /* comparisons: a NaN passes through */
        uc = u > limit ? limit : (u < -limit ? -limit : u);
    }
    return (gc / (1.0f + expf(-gc))) * uc;
}

float t3o_swiglu_clamped_out(float g, float u, float limit) {
    const float sg = g / (1.0f + expf(-g));
    if (limit <= 0.0f) return sg * u;
    const float sc = sg > limit ? limit : sg;
    const float uc = u > limit ? limit : (u < -limit ? -limit : u);
    return sc * uc;
}

int t3o_moe_row_clamped_at(const t3o_bank* b, int codebook, uint32_t mask, float limit, int clamp_at,
                           const float* x, const int32_t* slots, const float* scores, size_t topk, float* y,
                           size_t hits[3]) {
    const size_t hidden = b->hidden, inter = b->inter;
    const size_t gu_stride = (hidden / 16u) * (inter / 16u) * b->n_gu;
    const size_t dn_stride = (hidden / 16u) * (inter / 16u) * b->n_dn;
    float* gate_y = (float*)malloc(inter * sizeof(float));
    float* up_y = (float*)malloc(inter * sizeof(float));
    float* h = (float*)malloc(inter * sizeof(float));
    float* down_y = (float*)malloc(hidden * sizeof(float));
    if (!gate_y || !up_y || !h || !down_y) {
        free(gate_y);
        free(up_y);
        free(h);
        free(down_y);
        return -1;
    }
    size_t hit_gate = 0, hit_up = 0, total = 0;
    memset(y, 0, hidden * sizeof(float));
    for (size_t k = 0; k < topk; ++k) {
        if (slots[k] < 0 || (size_t)slots[k] >= b->experts) continue;
        const size_t e = (size_t)slots[k];
        t3o_project(x, b->gate_t + e * gu_stride, b->gate_suh + e * hidden, b->gate_svh + e * inter, hidden, inter,
                    b->n_gu, codebook, mask, gate_y);
        t3o_project(x, b->up_t + e * gu_stride, b->up_suh + e * hidden, b->up_svh + e * inter, hidden, inter,
                    b->n_gu, codebook, mask, up_y);
        for (size_t i = 0; i < inter; ++i) {
            h[i] = clamp_at == T3O_CLAMP_SILU_OUT ? t3o_swiglu_clamped_out(gate_y[i], up_y[i], limit)
                                                  : t3o_swiglu_clamped(gate_y[i], up_y[i], limit);
            if (limit > 0.0f) {
                const float gv = clamp_at == T3O_CLAMP_SILU_OUT ? gate_y[i] / (1.0f + expf(-gate_y[i])) : gate_y[i];
                hit_gate += gv > limit;
                hit_up += fabsf(up_y[i]) > limit;
            }
        }
        total += inter;
        t3o_project(h, b->down_t + e * dn_stride, b->down_suh + e * inter, b->down_svh + e * hidden, inter, hidden,
                    b->n_dn, codebook, mask, down_y);
        const float w = scores[k];
        for (size_t i = 0; i < hidden; ++i) y[i] += w * down_y[i];
    }
    if (hits) {
        hits[0] = hit_gate;
        hits[1] = hit_up;
        hits[2] = total;
    }
    free(gate_y);
    free(up_y);
    free(h);
    free(down_y);
    return 0;
}

double t3o_compare(const float* got, const float* ref, size_t len, double half_ulp) {
    double max_abs = 0.0, ss = 0.0;
    for (size_t i = 0; i < len; ++i) {
        const double d = fabs((double)got[i] - (double)ref[i]) - half_ulp * fabs((double)ref[i]);
        if (d > max_abs || d != d) max_abs = d;
        ss += (double)ref[i] * (double)ref[i];
    }
    const double rms = sqrt(ss / (double)len);
    return rms > 0.0 ? max_abs / rms : max_abs;
}

/* ---- the reference's launch-plan partitions (src/hip/plan.zig:86-109,249-260) ---------------------------- */

uint32_t t3o_rb_cap(uint32_t rows, uint32_t cap) {
    const uint32_t chunks = (rows + cap - 1u) / cap;
    return (rows + chunks - 1u) / chunks;
}
uint32_t t3o_bt_for(uint32_t rb) { return rb == 1u ? 4u : (rb <= 4u ? 2u : 1u); }
uint32_t t3o_ks_for(uint32_t in_f, uint32_t out_f) {
    const uint32_t q = (in_f / 16u) / 4u, groups = (out_f / 16u) / 4u;
    for (uint32_t d = 1; d <= q; ++d)
        if (q % d == 0 && groups * d >= 160u) return d;
    return q;
}
uint32_t t3o_ks_gu(uint32_t hidden, uint32_t ks_max) {
    uint32_t k = ks_max;
    while (k > 1u && (hidden / 16u) % (k * 2u) != 0u) k /= 2u;
    return k;
}
uint32_t t3o_ks_dn(uint32_t inter, uint32_t ks_max) {
    uint32_t k = ks_max;
    while (k > 1u && ((inter / 16u) % (k * 4u) != 0u || (inter / 16u) / (k * 4u) < 2u)) k /= 2u;
    return k;
}
