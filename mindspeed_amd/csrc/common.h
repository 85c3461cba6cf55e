// Shared helpers for the gfx950 kernels: error reporting, dtype conversion,
// 16-byte vector access.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/mindspeed_amd.h"

namespace ms {

// 16-byte vector as a native clang vector (usable with the nontemporal builtins).
typedef unsigned int v16 __attribute__((ext_vector_type(4)));

// Streaming (non-temporal) access for data that is touched once.
#define MS_NT_LOAD(p) __builtin_nontemporal_load(p)
#define MS_NT_STORE(v, p) __builtin_nontemporal_store((v), (p))

// ---- host-side error plumbing ------------------------------------------------
void set_error(const char *fmt, ...);

#define MS_REQUIRE(cond, code, ...)      \
    do {                                 \
        if (!(cond)) {                   \
            ms::set_error(__VA_ARGS__);  \
            return (code);               \
        }                                \
    } while (0)

#define MS_CHECK_LAUNCH(what)                                                     \
    do {                                                                          \
        hipError_t e_ = hipGetLastError();                                        \
        if (e_ != hipSuccess) {                                                   \
            ms::set_error("%s: launch failed: %s", (what), hipGetErrorString(e_)); \
            return MS_ERR_HIP;                                                    \
        }                                                                         \
    } while (0)

// hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, bytes), issued once per kernel and device
// (and again only if a larger size is asked for); later calls are a table lookup.  Returns a hipError_t.
hipError_t set_max_dynamic_lds(const void *fn, int bytes);

inline bool aligned16(const void *p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
inline int dtype_size(int dtype) { return dtype == MS_FP32 ? 4 : 2; }

// ---- device-side dtype helpers -----------------------------------------------
struct BF16 {
    using storage = uint16_t;
    static __device__ __forceinline__ float to_float(uint16_t v) {
        return __uint_as_float(static_cast<uint32_t>(v) << 16);
    }
    static __device__ __forceinline__ uint16_t from_float(float f) {
        __bf16 b = static_cast<__bf16>(f);  // round-to-nearest-even, NaN preserved
        return __builtin_bit_cast(uint16_t, b);
    }
};

struct FP16 {
    using storage = uint16_t;
    static __device__ __forceinline__ float to_float(uint16_t v) {
        return static_cast<float>(__builtin_bit_cast(_Float16, v));
    }
    static __device__ __forceinline__ uint16_t from_float(float f) {
        _Float16 h = static_cast<_Float16>(f);
        return __builtin_bit_cast(uint16_t, h);
    }
};

struct FP32 {
    using storage = float;
    static __device__ __forceinline__ float to_float(float v) { return v; }
    static __device__ __forceinline__ float from_float(float f) { return f; }
};

// A 16-byte vector of DT elements, convertible to / from floats.
template <typename DT>
struct Vec16 {
    static constexpr int N = 16 / sizeof(typename DT::storage);
    v16 raw;
    __device__ __forceinline__ void unpack(float *f) const {
        const typename DT::storage *p = reinterpret_cast<const typename DT::storage *>(&raw);
#pragma unroll
        for (int i = 0; i < N; ++i) f[i] = DT::to_float(p[i]);
    }
    __device__ __forceinline__ void pack(const float *f) {
        typename DT::storage *p = reinterpret_cast<typename DT::storage *>(&raw);
#pragma unroll
        for (int i = 0; i < N; ++i) p[i] = DT::from_float(f[i]);
    }
};

// Load a per-row scalar (probability) of runtime dtype as float.
__device__ __forceinline__ float load_scalar_as_float(const void *p, int64_t i, int dtype) {
    if (dtype == MS_FP32) return reinterpret_cast<const float *>(p)[i];
    uint16_t v = reinterpret_cast<const uint16_t *>(p)[i];
    return dtype == MS_BF16 ? BF16::to_float(v) : FP16::to_float(v);
}
__device__ __forceinline__ void store_float_as(void *p, int64_t i, int dtype, float f) {
    if (dtype == MS_FP32) {
        reinterpret_cast<float *>(p)[i] = f;
    } else {
        reinterpret_cast<uint16_t *>(p)[i] = dtype == MS_BF16 ? BF16::from_float(f) : FP16::from_float(f);
    }
}

}  // namespace ms
