// The plain f16 GEMM of the dense W_hat path (the role MLX's matmul has in turboexl3 src/core/dense.zig:1290-1302):
// rocBLAS, found at run time. The library is opened on the first call that wants it and never linked: a host without
// it keeps every other path, and the dense prefill then stays on the trellis GEMM.

#include <dlfcn.h>
#include <rocblas/rocblas.h>

#include <mutex>

#include "t3_host.hpp"

namespace t3 {
namespace {

struct Blas {
    void* lib = nullptr;
    rocblas_handle handle = nullptr;
    decltype(&rocblas_create_handle) create = nullptr;
    decltype(&rocblas_set_stream) set_stream = nullptr;
    decltype(&rocblas_set_pointer_mode) set_pointer_mode = nullptr;
    rocblas_status (*gemm_ex)(rocblas_handle, rocblas_operation, rocblas_operation, rocblas_int, rocblas_int,
                              rocblas_int, const void*, const void*, rocblas_datatype, rocblas_int, const void*,
                              rocblas_datatype, rocblas_int, const void*, const void*, rocblas_datatype, rocblas_int,
                              void*, rocblas_datatype, rocblas_int, rocblas_datatype, rocblas_gemm_algo, int32_t,
                              uint32_t) = nullptr;
    bool ok = false;
    std::mutex mutex;  // one handle, one stream setting a call
};

Blas& blas() {
    static Blas b;
    static std::once_flag once;
    std::call_once(once, [] {
        for (const char* name : {"librocblas.so.5", "librocblas.so", "/opt/rocm/lib/librocblas.so"}) {
            b.lib = dlopen(name, RTLD_NOW | RTLD_LOCAL);
            if (b.lib) break;
        }
        if (!b.lib) return;
        b.create = reinterpret_cast<decltype(b.create)>(dlsym(b.lib, "rocblas_create_handle"));
        b.set_stream = reinterpret_cast<decltype(b.set_stream)>(dlsym(b.lib, "rocblas_set_stream"));
        b.set_pointer_mode = reinterpret_cast<decltype(b.set_pointer_mode)>(dlsym(b.lib, "rocblas_set_pointer_mode"));
        b.gemm_ex = reinterpret_cast<decltype(b.gemm_ex)>(dlsym(b.lib, "rocblas_gemm_ex"));
        if (!b.create || !b.set_stream || !b.set_pointer_mode || !b.gemm_ex) return;
        if (b.create(&b.handle) != rocblas_status_success) return;
        b.set_pointer_mode(b.handle, rocblas_pointer_mode_host);
        b.ok = true;
    });
    return b;
}

}  // namespace

bool blas_available() { return blas().ok; }

// y [rows][cols] = x [rows][in] * w [in][cols of ldw], all f16 or all bf16, f32 accumulation, on `s`. Row-major
// operands are the column-major (cols x in, leading dimension ldw) and (in x rows) of a plain N, N product.
int32_t blas_gemm_half(hipStream_t s, bool bf16, const void* x, const void* w, uint32_t ldw, void* y, uint32_t rows,
                       uint32_t in, uint32_t cols) {
    Blas& b = blas();
    if (!b.ok) return T3_Exl3EngineNotImplemented;
    const float one = 1.0f, zero = 0.0f;
    const rocblas_datatype dt = bf16 ? rocblas_datatype_bf16_r : rocblas_datatype_f16_r;
    std::lock_guard<std::mutex> lock(b.mutex);
    if (b.set_stream(b.handle, s) != rocblas_status_success) return T3_HipFailed;
    const rocblas_status st = b.gemm_ex(
        b.handle, rocblas_operation_none, rocblas_operation_none, static_cast<rocblas_int>(cols),
        static_cast<rocblas_int>(rows), static_cast<rocblas_int>(in), &one, w, dt, static_cast<rocblas_int>(ldw), x, dt,
        static_cast<rocblas_int>(in), &zero, y, dt, static_cast<rocblas_int>(cols), y, dt,
        static_cast<rocblas_int>(cols), rocblas_datatype_f32_r, rocblas_gemm_algo_standard, 0, 0);
    return st == rocblas_status_success ? T3_OK : T3_HipFailed;
}

// z f16 [rows][out] = xp f16 [rows][in] * w_hat f16 [in][out]
int32_t blas_gemm_f16(hipStream_t s, const uint16_t* xp, const uint16_t* w_hat, uint16_t* z, uint32_t rows, uint32_t in,
                      uint32_t out) {
    return blas_gemm_half(s, false, xp, w_hat, out, z, rows, in, out);
}

}  // namespace t3
