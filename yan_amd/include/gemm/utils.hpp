// Small compile-time helpers and vector types shared by the gfx950 GEMM kernels.
// Counterpart of the reference's yan/include/gemm/utils.cuh:5-13 (ceil_div, constexpr_gcd).
#pragma once

#include <hip/hip_runtime.h>
#include <cstdint>

namespace yan {

template <typename T>
__host__ __device__ constexpr T ceil_div(T a, T b) { return (a + b - 1) / b; }

template <typename T>
__host__ __device__ constexpr T constexpr_gcd(T a, T b) { return b == 0 ? a : constexpr_gcd(b, a % b); }

typedef float    f32x4  __attribute__((ext_vector_type(4)));
typedef float    f32x16 __attribute__((ext_vector_type(16)));
typedef int      i32x4  __attribute__((ext_vector_type(4)));
typedef int      i32x8  __attribute__((ext_vector_type(8)));
typedef __bf16   bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16   bf16x8 __attribute__((ext_vector_type(8)));
typedef _Float16 f16x4  __attribute__((ext_vector_type(4)));
typedef _Float16 f16x8  __attribute__((ext_vector_type(8)));

constexpr int kWaveSize  = 64;
constexpr int kRowBytes  = 128;   // one LDS tile row: 64 bf16/fp16 or 128 fp8 values along K
constexpr int kChunk     = 16;    // bytes moved per lane per memory instruction
constexpr int kNumXCD    = 8;     // MI355X: 8 accelerator dies, 32 CUs and one 4 MB L2 each

#define YAN_GLOBAL_PTR(p) ((const __attribute__((address_space(1))) void*)(p))
#define YAN_LDS_PTR(p)    ((__attribute__((address_space(3))) void*)(p))

// s_waitcnt immediates on gfx9: vmcnt = bits [3:0] | [15:14], expcnt [6:4], lgkmcnt [11:8].
__host__ __device__ constexpr int waitcnt_imm(int vmcnt, int lgkmcnt) {
    return (vmcnt & 0xf) | ((vmcnt >> 4) << 14) | (0x7 << 4) | ((lgkmcnt & 0xf) << 8);
}
constexpr int kNoWaitVm   = 63;
constexpr int kNoWaitLgkm = 15;

// Compute units of the current device (256 on MI355X), asked once per process; 256 if the runtime will not say.
inline int device_cu_count() {
    static const int cus = [] {
        int device = 0, count = 0;
        if (hipGetDevice(&device) != hipSuccess ||
            hipDeviceGetAttribute(&count, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || count < kNumXCD)
            count = 256;
        return count;
    }();
    return cus;
}

} // namespace yan
