// Shared helpers of the gfx950 kernels behind include/dmoe.h.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include "../../include/dmoe.h"

namespace dmoe {

constexpr int kWave = 64;  // CDNA wavefront width

// Thread-local message returned by dmoe_last_error().
char *error_buffer();
int fail(int code, const char *fmt, ...);

#define DMOE_REQUIRE(cond, code, ...)            \
    do {                                         \
        if (!(cond)) return ::dmoe::fail((code), __VA_ARGS__); \
    } while (0)

#define DMOE_HIP(expr)                                                              \
    do {                                                                            \
        hipError_t err__ = (expr);                                                  \
        if (err__ != hipSuccess)                                                    \
            return ::dmoe::fail(DMOE_ERR_HIP, "%s: %s", #expr, hipGetErrorString(err__)); \
    } while (0)

// Launch errors (bad configuration) surface here; execution stays asynchronous.
#define DMOE_LAUNCH_CHECK(name)                                                     \
    do {                                                                            \
        hipError_t err__ = hipGetLastError();                                       \
        if (err__ != hipSuccess)                                                    \
            return ::dmoe::fail(DMOE_ERR_HIP, "launch of %s: %s", (name), hipGetErrorString(err__)); \
    } while (0)

int device_cus();  // compute units of the current device, cached per device

// Raises a kernel's dynamic LDS limit to `bytes` on the current device, once per device: `seen` is the caller's
// record of the devices done (a static, one per kernel).  Serialised, and a device is recorded only after the call
// succeeded, so no thread launches before the attribute is in place and a failure is retried by the next launch.
hipError_t raise_dynamic_lds(const void *kernel, int bytes, unsigned long long *seen);

__device__ __forceinline__ int lane_id() { return threadIdx.x & (kWave - 1); }

// bf16 <-> fp32, round to nearest even (NaN kept quiet).
__device__ __forceinline__ float bf16_to_f32(uint16_t v) { return __uint_as_float(((uint32_t)v) << 16); }
__device__ __forceinline__ uint16_t f32_to_bf16(float f) {
    uint32_t u = __float_as_uint(f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40u);
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
    // gfx950 converts a pair in one instruction (v_cvt_pk_bf16_f32, round to nearest even)
    typedef float f32x2_t __attribute__((ext_vector_type(2)));
    typedef __bf16 bf16x2_t __attribute__((ext_vector_type(2)));
    const f32x2_t v = {lo, hi};
    const bf16x2_t r = __builtin_convertvector(v, bf16x2_t);
    uint32_t u;
    __builtin_memcpy(&u, &r, 4);
    return u;
}
// silu(g) * u on fp32 with the hardware exponential and reciprocal (about 1 ulp each)
__device__ __forceinline__ float silu_mul(float g, float u) {
    return g * __builtin_amdgcn_rcpf(1.f + __expf(-g)) * u;
}

}  // namespace dmoe
