// Per-head batched GEMM mhd[m,h,:] = mht[m,h,:t] @ w[h] used around the MLA attention
// (W_UK absorb and W_UV projection). Replaces XliteOpEinsumMhtHtdMhd / XliteOpEinsumMhtHdtMhd
// (xlite/csrc/op.cpp:1872-1918, kernels/einsum_mht_htd_mhd.h:9-37).
//
// One wave computes a 32 x 32 output tile with v_mfma_f32_32x32x16, operands straight from
// global memory (the left operand rows are k-contiguous; the [h,t,d] weight is read with
// 2-byte loads that are contiguous across lanes). A workgroup covers 32 rows x 128 columns.
#include "common.h"

namespace xlite {

namespace {

template <typename T>
struct Mma;
template <>
struct Mma<BF16> {
    static __device__ __forceinline__ f32x16_t run(const uint4 &a, const uint4 &b, f32x16_t c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a),
                                                       __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
    }
};
template <>
struct Mma<FP16> {
    static __device__ __forceinline__ f32x16_t run(const uint4 &a, const uint4 &b, f32x16_t c)
    {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a),
                                                      __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
    }
};

template <typename T, bool HDT>
__global__ void __launch_bounds__(256)
einsum_kernel(const uint16_t *__restrict__ mht, const uint16_t *__restrict__ w,
              uint16_t *__restrict__ mhd, uint32_t m, uint32_t h, uint32_t t, uint32_t d,
              uint32_t t_stride)
{
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t col = lane & 31, half = lane >> 5;
    const uint32_t head = blockIdx.z;
    const uint32_t m0 = blockIdx.y * 32;
    const uint32_t n0 = blockIdx.x * 128 + wave * 32;
    if (n0 >= d) {
        return;
    }
    const uint32_t row = m0 + col;
    const bool row_ok = row < m;
    const uint16_t *a_ptr = mht + (static_cast<uint64_t>(row_ok ? row : 0) * h + head) * t_stride;
    const uint16_t *w_head = w + static_cast<uint64_t>(head) * t * d;
    const uint32_t n = n0 + col;

    f32x16_t acc;
#pragma unroll
    for (int k = 0; k < 16; k++) {
        acc[k] = 0.f;
    }
    for (uint32_t k0 = 0; k0 < t; k0 += 16) {
        const uint32_t kk = k0 + half * 8;
        uint4 a = make_uint4(0, 0, 0, 0);
        if (row_ok) {
            a = *reinterpret_cast<const uint4 *>(a_ptr + kk);
        }
        uint4 b;
        if (HDT) {
            b = *reinterpret_cast<const uint4 *>(w_head + static_cast<uint64_t>(n) * t + kk);
        } else {
            uint16_t e[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                e[i] = w_head[static_cast<uint64_t>(kk + i) * d + n];
            }
            b.x = e[0] | (static_cast<uint32_t>(e[1]) << 16);
            b.y = e[2] | (static_cast<uint32_t>(e[3]) << 16);
            b.z = e[4] | (static_cast<uint32_t>(e[5]) << 16);
            b.w = e[6] | (static_cast<uint32_t>(e[7]) << 16);
        }
        acc = Mma<T>::run(a, b, acc);
    }
    // C[i][j]: j = lane % 32 (column n), i = 8 * (k / 4) + 4 * (lane / 32) + k % 4 (row)
#pragma unroll
    for (int k = 0; k < 16; k++) {
        const uint32_t r = m0 + (k / 4) * 8 + half * 4 + (k % 4);
        if (r < m) {
            mhd[(static_cast<uint64_t>(r) * h + head) * d + n] = T::from_f32(acc[k]);
        }
    }
}

}  // namespace
}  // namespace xlite

using namespace xlite;

extern "C" int xlite_hip_einsum_mht_mhd(void *stream, const void *mht, const void *w, void *mhd,
                                        uint32_t m, uint32_t h, uint32_t t, uint32_t d,
                                        uint32_t t_stride, int w_is_hdt, int dtype)
{
    XL_REQUIRE(dtype == XLITE_HIP_BF16 || dtype == XLITE_HIP_FP16, "mht/w/mhd dtype unsupported!");
    if (m == 0 || h == 0) {
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(mht && w && mhd, "null tensor");
    XL_REQUIRE(t % 16 == 0 && t > 0, "t must be a positive multiple of 16");
    XL_REQUIRE(d % 32 == 0 && d > 0, "d must be a positive multiple of 32");
    XL_REQUIRE(t_stride >= t && t_stride % 8 == 0, "t_stride must be >= t and a multiple of 8");
    if (m == 0 || h == 0) {
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(h <= 65535 && ceil_div(m, 32) <= 65535, "grid too large");
    dim3 grid(ceil_div(d, 128), ceil_div(m, 32), h);
    hipStream_t s = as_stream(stream);
    const uint16_t *a = static_cast<const uint16_t *>(mht);
    const uint16_t *b = static_cast<const uint16_t *>(w);
    uint16_t *c = static_cast<uint16_t *>(mhd);
    if (dtype == XLITE_HIP_BF16) {
        if (w_is_hdt) {
            einsum_kernel<BF16, true><<<grid, 256, 0, s>>>(a, b, c, m, h, t, d, t_stride);
        } else {
            einsum_kernel<BF16, false><<<grid, 256, 0, s>>>(a, b, c, m, h, t, d, t_stride);
        }
    } else {
        if (w_is_hdt) {
            einsum_kernel<FP16, true><<<grid, 256, 0, s>>>(a, b, c, m, h, t, d, t_stride);
        } else {
            einsum_kernel<FP16, false><<<grid, 256, 0, s>>>(a, b, c, m, h, t, d, t_stride);
        }
    }
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}
