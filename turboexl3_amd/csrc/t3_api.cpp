// The C ABI of the gfx950 EXL3 projection engine (include/turboexl3_hip.h): validation with the reference's refusal
// names, this library's launch partitions and workspace layout, and the launches. Host logic only; the kernels live in
// the .hip files beside this one.

#include "../../include/turboexl3_hip.h"

#include <atomic>
#include <cstring>
#include <mutex>

#include "t3_host.hpp"

namespace {

// t3_configure writes the next slot of a small ring and then publishes its index, so a reader copies a whole snapshot
// also while another thread configures (a slot is reused only after 63 further t3_configure calls). An entry point
// copies the published snapshot ONCE, into its thread's own storage (ConfigScope), and everything it calls reads that
// copy: a call's checks, workspace carving and launches all see the same settings whatever another thread configures
// meanwhile. (The reference sets its configuration once before the first call, src/core/config.zig:175-178.)
constexpr uint32_t kConfigSlots = 64;
// what a process that never configures runs with, and what t3_config_default hands out
constexpr t3_config kDefaultConfig = {9, 1, 1, 0, 1, 513, 0};
t3_config g_configs[kConfigSlots] = {kDefaultConfig};
std::atomic<uint32_t> g_config_at{0};
std::mutex g_config_write;

thread_local t3_config tl_config = kDefaultConfig;
thread_local int tl_config_depth = 0;

t3_config published_config() { return g_configs[g_config_at.load(std::memory_order_acquire) % kConfigSlots]; }

}  // namespace

namespace t3 {

// the calling entry point's snapshot; outside any entry point (a helper called on its own), what is published now
const t3_config& config() {
    if (tl_config_depth == 0) tl_config = published_config();
    return tl_config;
}

ConfigScope::ConfigScope() {
    if (tl_config_depth++ == 0) tl_config = published_config();
}
ConfigScope::~ConfigScope() { --tl_config_depth; }

}  // namespace t3

extern "C" {

const char* t3_error_name(int32_t status) {
    switch (status) {
        case T3_OK: return "ok";
        case T3_BadExl3Shape: return "BadExl3Shape";
        case T3_BadExl3Dtype: return "BadExl3Dtype";
        case T3_Exl3EngineNotImplemented: return "Exl3EngineNotImplemented";
        case T3_Exl3EngineCacheFull: return "Exl3EngineCacheFull";
        case T3_Exl3GateUpRateMismatch: return "Exl3GateUpRateMismatch";
        case T3_InvalidExl3Clamp: return "InvalidExl3Clamp";
        case T3_Exl3TopKExceedsReduceBank: return "Exl3TopKExceedsReduceBank";
        case T3_Exl3WindowUnsupported: return "Exl3WindowUnsupported";
        case T3_ExpertLayoutUnsupported: return "ExpertLayoutUnsupported";
        case T3_InvalidTurboexl3Config: return "InvalidTurboexl3Config";
        case T3_WorkspaceTooSmall: return "WorkspaceTooSmall";
        case T3_HipFailed: return "HipFailed";
        case T3_BadArgs: return "BadArgs";
        case T3_NotExl3: return "NotExl3";
        case T3_Exl3CodebookUnsupported: return "Exl3CodebookUnsupported";
        case T3_Exl3RateUnsupported: return "Exl3RateUnsupported";
        case T3_MissingWeight: return "MissingWeight";
        case T3_Exl3TrellisGeometry: return "Exl3TrellisGeometry";
        case T3_Exl3WidthNotMultipleOf128: return "Exl3WidthNotMultipleOf128";
        case T3_Exl3SideGeometry: return "Exl3SideGeometry";
        case T3_Exl3SideDtype: return "Exl3SideDtype";
        default: return "UnknownStatus";
    }
}

void t3_config_default(t3_config* out) {
    if (!out) return;
    *out = kDefaultConfig;
}

int32_t t3_configure(const t3_config* cfg) {
    if (!cfg) return T3_BadArgs;
    const bool flags_ok = (cfg->dec_one == 0 || cfg->dec_one == 1) && (cfg->prefill == 0 || cfg->prefill == 1) &&
                          (cfg->mcg_pair == 0 || cfg->mcg_pair == 1) && (cfg->mul1_defer == 0 || cfg->mul1_defer == 1) &&
                          cfg->dense_gemm_rows >= 0 && (cfg->dense_rows_alone == 0 || cfg->dense_rows_alone == 1);
    // the reference's own set (src/core/config.zig:140): any other value is refused, as there
    const int32_t f = cfg->decode_form;
    if ((f != 3 && f != 5 && f != 6 && f != 7 && f != 8 && f != 9) || !flags_ok) return T3_InvalidTurboexl3Config;
    std::lock_guard<std::mutex> lock(g_config_write);
    const uint32_t next = g_config_at.load(std::memory_order_relaxed) + 1u;
    g_configs[next % kConfigSlots] = *cfg;
    g_config_at.store(next, std::memory_order_release);
    return T3_OK;
}

void t3_release_engines(void) {}

int32_t t3_rate_admitted(int64_t n) { return t3::rate_ok(n) ? 1 : 0; }

int32_t t3_admit_topk(int64_t topk) { return topk > T3_REDUCE_MAX_TOPK ? T3_Exl3TopKExceedsReduceBank : T3_OK; }

int32_t t3_trellis_admitted(const int64_t* shape, int32_t ndim, int64_t experts, int64_t in_dim, int64_t out_dim,
                            int64_t n_max) {
    if (!shape || ndim != 4) return 0;
    for (int i = 0; i < 4; ++i)
        if (shape[i] <= 0) return 0;
    if (in_dim % 16 != 0 || out_dim % 16 != 0) return 0;
    if (shape[0] != experts || shape[1] != in_dim / 16 || shape[2] != out_dim / 16) return 0;
    if (!t3::rate_ok(shape[3])) return 0;
    return shape[3] <= n_max ? 1 : 0;
}

int32_t t3_test_codebooks(t3_stream stream, uint16_t* mcg, uint16_t* mul1, uint16_t* t) {
    if (!mcg || !mul1 || !t) return T3_BadArgs;
    return t3::hip_status(t3::launch_test_codebooks(mcg, mul1, t, static_cast<hipStream_t>(stream)));
}

int32_t t3_test_lane(t3_stream stream, const uint16_t* trellis, int64_t n, int32_t window_bits, int64_t tiles,
                     uint16_t* cw, uint16_t* mcg, uint16_t* mul1) {
    if (!trellis || !cw || !mcg || !mul1) return T3_BadArgs;
    if (!t3::rate_ok(n) || tiles <= 0 || tiles > (1 << 24)) return T3_BadExl3Shape;
    if (window_bits < 8 || window_bits > 16) return T3_Exl3WindowUnsupported;
    return t3::hip_status(t3::launch_test_lane(reinterpret_cast<const uint32_t*>(trellis), static_cast<uint32_t>(n),
                                               static_cast<uint32_t>(window_bits), static_cast<uint32_t>(tiles), cw, mcg,
                                               mul1, static_cast<hipStream_t>(stream)));
}

int32_t t3_test_convert(t3_stream stream, const float* in, uint16_t* bf16, uint16_t* f16, float* back, int64_t count) {
    if (!in || !bf16 || !f16 || !back) return T3_BadArgs;
    if (count <= 0 || count > (1 << 28)) return T3_BadExl3Shape;
    return t3::hip_status(t3::launch_test_convert(in, bf16, f16, back, static_cast<uint32_t>(count),
                                                  static_cast<hipStream_t>(stream)));
}

int32_t t3_test_hbm_read(t3_stream stream, const void* src, uint64_t bytes, uint32_t* sink, int32_t workgroups) {
    if (!src || !sink) return T3_BadArgs;
    if (bytes == 0 || bytes % 16u != 0u || (reinterpret_cast<uintptr_t>(src) & 15u) != 0u || workgroups <= 0 ||
        workgroups > (1 << 20))
        return T3_BadExl3Shape;
    return t3::hip_status(t3::launch_test_hbm_read(src, bytes, sink, static_cast<uint32_t>(workgroups),
                                                   static_cast<hipStream_t>(stream)));
}

int32_t t3_test_mfma(t3_stream stream, const uint16_t* a, const uint16_t* b, float* d) {
    if (!a || !b || !d) return T3_BadArgs;
    return t3::hip_status(t3::launch_test_mfma(a, b, d, static_cast<hipStream_t>(stream)));
}

}  // extern "C"
