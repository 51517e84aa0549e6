// Routed experts: `moe`, `moeClamped`, `moeWithShared` (turboexl3 src/root.zig:822-904,976-1004).

#include "t3_host.hpp"

extern "C" {

int32_t t3_moe_workspace_bytes(const t3_array*, const t3_bank*, const t3_array*, size_t*) {
    return T3_Exl3EngineNotImplemented;
}

int32_t t3_moe(t3_stream, const t3_array*, const t3_bank*, const t3_array*, const t3_array*, t3_decode, int32_t,
               t3_array*, void*, size_t) {
    return T3_Exl3EngineNotImplemented;
}

int32_t t3_moe_clamped(t3_stream, const t3_array*, const t3_bank*, const t3_array*, const t3_array*, t3_decode,
                       int32_t, t3_array*, void*, size_t) {
    return T3_Exl3EngineNotImplemented;
}

int32_t t3_moe_with_shared(t3_stream, const t3_array*, const t3_bank*, const t3_array*, const t3_array*, t3_decode,
                           int32_t, const t3_array*, t3_array*, void*, size_t) {
    return T3_Exl3EngineNotImplemented;
}

}  // extern "C"
