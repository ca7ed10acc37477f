// Shared device/host helpers for the gfx950 LSTM kernels.
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <cstddef>
#include <cstdint>

namespace flstm_hip {

typedef _Float16 half_t;
typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef _Float16 half4 __attribute__((ext_vector_type(4)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef unsigned long long u64;

constexpr int kWave = 64;

__host__ __device__ inline size_t round_up(size_t v, size_t m) { return (v + m - 1) / m * m; }
__host__ __device__ inline size_t ceil_div(size_t v, size_t m) { return (v + m - 1) / m; }

// 16-byte global load of eight fp16 values (address must be 16-byte aligned).
__device__ __forceinline__ half8 ld_half8(const half_t* p) {
    return *reinterpret_cast<const half8*>(p);
}
__device__ __forceinline__ void st_half8(half_t* p, half8 v) {
    *reinterpret_cast<half8*>(p) = v;
}

// Eight fp16 values fetched with two 8-byte device-scope relaxed atomic loads.  These bypass the
// per-CU vector L1 and are served by the L2 of the XCD, so data stored by another CU of the same
// XCD (plain write-through stores) or by any CU (device-scope atomic stores) is observed without
// a cache invalidate.
__device__ __forceinline__ half8 ld_half8_coherent(const half_t* p) {
    union { u64 q[2]; half8 h; } u;
    u.q[0] = __hip_atomic_load(reinterpret_cast<const u64*>(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    u.q[1] = __hip_atomic_load(reinterpret_cast<const u64*>(p) + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    return u.h;
}

__device__ __forceinline__ float sigmoidf_dev(float x) { return 1.0f / (1.0f + __expf(-x)); }
__device__ __forceinline__ float tanhf_dev(float x) {
    // tanh(x) = 2*sigmoid(2x) - 1, evaluated with the hardware exp; absolute error ~1e-7.
    return 2.0f / (1.0f + __expf(-2.0f * x)) - 1.0f;
}

}  // namespace flstm_hip
