// Host-side launch descriptors of the kernel groups; the C ABI (t3_api.cpp) fills them after validation.
#pragma once

#include <hip/hip_runtime.h>

#include <cstddef>
#include <cstdint>

namespace t3 {

// One dense projection call. Buffers by role, as the reference's HIP plan names them (turboexl3
// src/hip/plan.zig:9-45): x, suh, svh, trellis, and the scratch xq (prepared rows), xs (block sums), z (planes).
struct DenseLaunch {
    const void* x = nullptr;
    const uint16_t* suh = nullptr;
    const uint16_t* svh = nullptr;
    const uint32_t* trellis = nullptr;
    uint32_t* xq = nullptr;
    float* xs = nullptr;
    float* z = nullptr;
    void* y = nullptr;
    uint32_t* arrive = nullptr;  // the fused launch's arrival counters
    uint32_t in = 0, out = 0, rows = 0, n = 0, wbits = 16;
    int codebook = 0;  // t3::Codebook
    int dtype = 0;     // t3::Dtype of x and y
    uint32_t ks = 1, bt = 4;
};

// the GEMV launch's form: 0 planes only (the chain), 1 + the finish by the last workgroup to arrive at a column block,
// 2 + the prepare inside the launch (up to 4 rows)
enum DenseFuse : int { kFuseChain = 0, kFuseArrive = 1, kFuseOne = 2 };

hipError_t launch_dense_prep(const DenseLaunch& d, hipStream_t s);
hipError_t launch_dense_gemv(const DenseLaunch& d, int fuse, hipStream_t s);
hipError_t launch_dense_finish(const DenseLaunch& d, hipStream_t s);

// trellis [in/16][out/16][n] -> W_hat f16 [in][out], bit-exact (format.reconstructInner)
hipError_t launch_dequant(const uint32_t* trellis, uint16_t* w_hat, uint32_t in, uint32_t out, uint32_t n,
                          uint32_t wbits, int codebook, hipStream_t s);

// test kernels: every codeword's MCG and MUL1 value and MUL1 byte sum; every tile's 256 codewords by code position
hipError_t launch_test_codebooks(uint16_t* mcg, uint16_t* mul1, uint16_t* t, hipStream_t s);
hipError_t launch_test_lane(const uint32_t* trellis, uint32_t n, uint32_t wbits, uint32_t tiles, uint16_t* cw,
                            uint16_t* mcg, uint16_t* mul1, hipStream_t s);
// test kernel: D = A B through the GEMV's MFMA with the fragments the kernels assume
hipError_t launch_test_mfma(const uint16_t* a, const uint16_t* b, float* d, hipStream_t s);

}  // namespace t3
