// Shared host/device helpers of the gfx950 attention library.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>

#include <string>

#include "../../include/xlite_hip.h"

namespace xlite {

// ---- error plumbing ---------------------------------------------------------
void set_error(const std::string &msg);
int fail(int code, const char *func, const std::string &msg);
// allows `bytes` of dynamic LDS for `kernel` on the current device (once per kernel, device and size)
int ensure_dynamic_lds(const void *kernel, size_t bytes);
// device buffer of four 64-bit words set through xlite_hip_set_clock_probe, or nullptr (the usual case)
unsigned long long *clock_probe();

#define XL_REQUIRE(cond, msg)                                                      \
    do {                                                                           \
        if (!(cond)) {                                                             \
            return ::xlite::fail(XLITE_HIP_EINVAL, __func__, std::string(msg));    \
        }                                                                          \
    } while (0)

#define XL_HIP(expr)                                                               \
    do {                                                                           \
        hipError_t _e = (expr);                                                    \
        if (_e != hipSuccess) {                                                    \
            return ::xlite::fail(XLITE_HIP_ERUNTIME, __func__,                     \
                                 std::string(#expr) + ": " + hipGetErrorString(_e)); \
        }                                                                          \
    } while (0)

// Launch errors (bad configuration) surface through hipGetLastError.
#define XL_LAUNCH_CHECK() XL_HIP(hipGetLastError())

inline hipStream_t as_stream(void *s) { return reinterpret_cast<hipStream_t>(s); }

__host__ __device__ static inline uint32_t ceil_div(uint32_t a, uint32_t b) { return (a + b - 1) / b; }

// ---- device-side 16-bit float helpers ----------------------------------------
typedef __attribute__((__vector_size__(2 * sizeof(__bf16)))) __bf16 bf16x2_t;
typedef __attribute__((__vector_size__(8 * sizeof(__bf16)))) __bf16 bf16x8_t;
typedef __attribute__((__vector_size__(2 * sizeof(_Float16)))) _Float16 f16x2_t;
typedef __attribute__((__vector_size__(8 * sizeof(_Float16)))) _Float16 f16x8_t;
typedef __attribute__((__vector_size__(4 * sizeof(float)))) float f32x4_t;
typedef __attribute__((__vector_size__(16 * sizeof(float)))) float f32x16_t;

struct BF16 {
    static constexpr int kCode = XLITE_HIP_BF16;
    typedef __bf16 elem;
    typedef bf16x2_t pair;
    static __device__ __forceinline__ float to_f32(uint16_t h)
    {
        return __builtin_bit_cast(float, static_cast<uint32_t>(h) << 16);
    }
    // round to nearest even, the conversion the reference kernels use (vconv_f322bf16r)
    static __device__ __forceinline__ uint16_t from_f32(float f)
    {
        return __builtin_bit_cast(uint16_t, static_cast<__bf16>(f));
    }
    static __device__ __forceinline__ float lo(uint32_t w) { return __builtin_bit_cast(float, w << 16); }
    static __device__ __forceinline__ float hi(uint32_t w)
    {
        return __builtin_bit_cast(float, w & 0xffff0000u);
    }
    static __device__ __forceinline__ uint32_t pack(float a, float b)
    {
        bf16x2_t r;
        r[0] = static_cast<__bf16>(a);
        r[1] = static_cast<__bf16>(b);
        return __builtin_bit_cast(uint32_t, r);
    }
    // a.lo*b.lo + a.hi*b.hi + c with fp32 accumulation (v_dot2_f32_bf16)
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c)
    {
        return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a),
                                               __builtin_bit_cast(bf16x2_t, b), c, false);
    }
};

struct FP16 {
    static constexpr int kCode = XLITE_HIP_FP16;
    typedef _Float16 elem;
    typedef f16x2_t pair;
    static __device__ __forceinline__ float to_f32(uint16_t h)
    {
        return static_cast<float>(__builtin_bit_cast(_Float16, h));
    }
    static __device__ __forceinline__ uint16_t from_f32(float f)
    {
        return __builtin_bit_cast(uint16_t, static_cast<_Float16>(f));
    }
    static __device__ __forceinline__ float lo(uint32_t w)
    {
        return to_f32(static_cast<uint16_t>(w & 0xffffu));
    }
    static __device__ __forceinline__ float hi(uint32_t w) { return to_f32(static_cast<uint16_t>(w >> 16)); }
    static __device__ __forceinline__ uint32_t pack(float a, float b)
    {
        f16x2_t r;
        r[0] = static_cast<_Float16>(a);
        r[1] = static_cast<_Float16>(b);
        return __builtin_bit_cast(uint32_t, r);
    }
    static __device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c)
    {
        return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, a), __builtin_bit_cast(f16x2_t, b),
                                      c, false);
    }
};

// ---- cross-lane helpers (DPP, no LDS traffic) -----------------------------------
// xor-1, xor-2 inside a quad; then mirror inside 8 and inside 16 lanes. Applied in this
// order to a value that is already uniform inside the smaller group, each step behaves
// like the matching butterfly exchange.
template <int CTRL>
__device__ __forceinline__ float dpp_f32(float v)
{
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, 0xF, 0xF, false));
}
constexpr int DPP_QUAD_XOR1 = 0xB1;       // quad_perm:[1,0,3,2]
constexpr int DPP_QUAD_XOR2 = 0x4E;       // quad_perm:[2,3,0,1]
constexpr int DPP_ROW_HALF_MIRROR = 0x141;
constexpr int DPP_ROW_MIRROR = 0x140;

// Sum over groups of LANES consecutive lanes (LANES in {1,2,4,8,16}); every lane of the
// group ends with the group's sum.
template <int LANES>
__device__ __forceinline__ float group_sum(float v)
{
    if constexpr (LANES >= 2) v += dpp_f32<DPP_QUAD_XOR1>(v);
    if constexpr (LANES >= 4) v += dpp_f32<DPP_QUAD_XOR2>(v);
    if constexpr (LANES >= 8) v += dpp_f32<DPP_ROW_HALF_MIRROR>(v);
    if constexpr (LANES >= 16) v += dpp_f32<DPP_ROW_MIRROR>(v);
    return v;
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

}  // namespace xlite
