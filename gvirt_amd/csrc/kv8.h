// Dequantisation of 8-bit cache values, shared by the copy that serves the 16-bit kernels (kv_dequant.hip) and by the
// prefill kernel that reads quantised caches itself (prefill_mfma.hip): the same code, so the two give the same bits.
#pragma once

#include "common.h"

namespace xlite {

__device__ __forceinline__ float clamp_f16(float x) { return fminf(fmaxf(x, -65504.f), 65504.f); }

template <typename T, int KVF>
__device__ __forceinline__ uint4 dequant8(const uint2 &raw, float scale)
{
    float x[8];
    if constexpr (KVF == XLITE_HIP_KV_INT8) {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int32_t b = static_cast<int8_t>(((j < 4 ? raw.x : raw.y) >> (8 * (j % 4))) & 0xffu);
            x[j] = static_cast<float>(b) * scale;
        }
    } else {
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const int w = static_cast<int>(j < 4 ? raw.x : raw.y);
            float f;
            switch (j % 4) {
            case 0: f = __builtin_amdgcn_cvt_f32_fp8(w, 0); break;
            case 1: f = __builtin_amdgcn_cvt_f32_fp8(w, 1); break;
            case 2: f = __builtin_amdgcn_cvt_f32_fp8(w, 2); break;
            default: f = __builtin_amdgcn_cvt_f32_fp8(w, 3); break;
            }
            x[j] = f * scale;
        }
    }
#pragma unroll
    for (int j = 0; j < 8; j++) {
        x[j] = clamp_f16(x[j]);
    }
    return make_uint4(T::pack(x[0], x[1]), T::pack(x[2], x[3]), T::pack(x[4], x[5]), T::pack(x[6], x[7]));
}

}  // namespace xlite
