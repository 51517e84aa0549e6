// Host-side helpers shared by the C ABI's translation units: descriptor checks, the decode descriptor, workspace
// carving and this library's launch partitions.
#pragma once

#include <cstddef>
#include <cstdint>

#include "../../include/turboexl3_hip.h"
#include "t3_kernels.hpp"

namespace t3 {

// The configuration the current call runs with. An entry point opens a ConfigScope first: the published configuration is
// copied once into the thread's own storage and every config() below it, however deep, reads that one copy.
const t3_config& config();
struct ConfigScope {
    ConfigScope();
    ~ConfigScope();
    ConfigScope(const ConfigScope&) = delete;
    ConfigScope& operator=(const ConfigScope&) = delete;
};

inline bool rate_ok(int64_t n) { return n % 2 == 0 && n >= 16 && n <= 128; }

inline int32_t hip_status(hipError_t e) { return e == hipSuccess ? T3_OK : T3_HipFailed; }

inline bool array_ok(const t3_array* a) {
    if (!a || !a->data || a->ndim < 0 || a->ndim > T3_MAX_DIMS) return false;
    for (int i = 0; i < a->ndim; ++i)
        if (a->shape[i] < 0) return false;
    return true;
}

// The kernels read activations, scale vectors and trellises 16 bytes a lane and carve the workspace in 256-byte steps:
// an array they touch that way starts on a 16-byte boundary, the workspace on a 256-byte one (what hipMalloc and any
// tensor library's allocations and whole-row views give).
inline bool aligned16(const t3_array* a) { return (reinterpret_cast<uintptr_t>(a->data) & 15u) == 0u; }
inline bool workspace_ok(const void* w) { return w && (reinterpret_cast<uintptr_t>(w) & 255u) == 0u; }

// Widths and row counts the launches index with 32-bit arithmetic and 16-bit grid dimensions: in / 16 is a grid's y
// where W_hat is decoded or un-rotated (at most 65535), and a call's rows x width addresses its scratch in 32 bits.
// Beyond them an entry point refuses with Exl3EngineNotImplemented before it launches anything.
inline bool widths_served(int64_t in, int64_t out) { return in / 16 <= 65535 && out <= (1ll << 24); }
inline bool rows_served(int64_t rows, int64_t in, int64_t out) {
    return rows * in < (1ll << 32) && rows * out < (1ll << 32);
}

inline bool is_act_dtype(int32_t d) { return d == T3_F32 || d == T3_F16 || d == T3_BF16; }
inline size_t dtype_size(int32_t d) { return d == T3_F32 || d == T3_U32 || d == T3_I32 ? 4 : 2; }

// The decode a call runs with: the reference's (codebook, window) plus this library's GEMV-only codebook forms.
struct Dec {
    int codebook;    // t3::Codebook numbering for exact decode (0 MUL1, 1 MCG)
    int gemv_form;   // the codebook the GEMV kernels run: exact, or kMul1Defer / kMcgPair by configuration
    uint32_t wbits;
};

inline int32_t resolve_decode(t3_decode dec, Dec* out) {
    if (dec.codebook != 0 && dec.codebook != 1) return T3_BadArgs;
    if (dec.window_bits < 8 || dec.window_bits > 16) return T3_Exl3WindowUnsupported;
    out->codebook = dec.codebook;
    out->wbits = static_cast<uint32_t>(dec.window_bits);
    if (dec.codebook == 1) out->gemv_form = config().mcg_pair ? 3 : 1;
    else out->gemv_form = config().mul1_defer ? 2 : 0;
    return T3_OK;
}

// Scratch carved from the caller's workspace in 256-byte steps.
struct Carver {
    unsigned char* base;
    size_t used = 0;
    explicit Carver(void* p) : base(static_cast<unsigned char*>(p)) {}
    template <typename T>
    T* take(size_t bytes) {
        T* p = base ? reinterpret_cast<T*>(base + used) : nullptr;
        used += (bytes + 255u) & ~static_cast<size_t>(255u);
        return p;
    }
};

// ---- partitions -----------------------------------------------------------------------------------------------
// The K split of a GEMV depends on the matrix's shape alone, never on the rows of a call, so a row's sums (and bytes)
// are those of the row alone. The reference fixes its split the same way (turboexl3 src/core/dense.zig:553-562); the
// numbers here are sized for 256 CUs, not for its 40-core target.

// output tiles a wave: one 128-bit load a lane covers a tile row's BT * 2n bytes (at most 1 KB)
inline uint32_t gemv_bt(uint32_t n) { return n <= 64u ? 8u : 4u; }
constexpr uint32_t kGemvTargetWgs = 768; // three workgroups a CU
constexpr uint32_t kGemvMinPer = 4;      // input tiles a wave at least

// K slices of a GEMV over in_tiles input tiles and `groups` workgroup columns: the smallest divisor d of
// in_tiles / 4 that reaches the target workgroup count while every wave keeps kGemvMinPer tiles. Splits that leave a
// wave whole 128-blocks of the input (per % 8 == 0) are preferred: the one-launch form prepares its input by block.
// Every split leaves a wave an even number of tiles: the f16-weight codebook forms walk two tile rows a step.
inline uint32_t gemv_slices(uint32_t in_tiles, uint32_t groups) {
    const uint32_t q = in_tiles / 4u;
    for (int whole = 1; whole >= 0; --whole) {
        uint32_t best = 0;
        for (uint32_t d = 1; d <= q; ++d) {
            if (q % d != 0) continue;
            const uint32_t per = q / d;
            if (per < kGemvMinPer && d > 1) break;
            if (per % 2u != 0u) continue;
            if (whole && per % 8u != 0u) continue;
            best = d;
            if (static_cast<uint64_t>(groups) * d >= kGemvTargetWgs) break;
        }
        if (best != 0) return best;
    }
    return 1;
}

// A dense GEMV's tiles a load and K slices. A small matrix cannot reach the target workgroup count at eight tiles a load
// (2560 x 640: 25 workgroups), and each of its few waves then walks its 64 tiles alone on a SIMD: with up to 128 workgroups
// the same rows are cut at four tiles a load, twice the workgroups of half the length. Measured (one row, us a call, eight
// against four tiles): 2560 x 640 8.2 / 7.1, 1024 x 4096 8.1 / 7.1, 2048 x 512 8.2 / 7.1, 2048 x 2048 8.4 / 8.0 (32 rows
// 11.2 / 9.9), 2048 x 4096 8.8 / 8.3; from about 144 workgroups up four tiles lose (4096 x 4096 9.6 / 10.0, 5120 x 5120
// 11.5 / 12.9). A column's sums do not depend on the tiles a load; the shape alone decides, so a row's bytes stay its own.
inline void dense_gemv_partition(uint32_t n, uint32_t in, uint32_t out, uint32_t* bt, uint32_t* ks) {
    *bt = gemv_bt(n);
    *ks = gemv_slices(in / 16u, (out / 16u) / *bt);
    if (*bt == 8u && (out / 128u) * *ks <= 128u) {
        *bt = 4u;
        *ks = gemv_slices(in / 16u, (out / 16u) / 4u);
    }
}

// The caller's workspace starts with the arrival counters of the fused launches, at a fixed place and size whatever
// the call's shapes: zero when the workspace is first passed, and zero again after every call.
constexpr size_t kCounterBytes = 65536;

}  // namespace t3
