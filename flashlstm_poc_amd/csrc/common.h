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

// Hardware exp2 / reciprocal (about 1 ulp each): absolute error of both functions is ~2e-7, far below
// the fp16 resolution of everything they feed.
__device__ __forceinline__ float sigmoidf_dev(float x) {
    return __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(-1.4426950408889634f * x));
}
__device__ __forceinline__ float tanhf_dev(float x) {
    // tanh(x) = 1 - 2 / (exp(2x) + 1); exp overflow gives 1 - 0, underflow gives 1 - 2
    return 1.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(2.8853900817779268f * x));
}

}  // namespace flstm_hip
