// Per-head batched GEMM mhd[m,h,:] = mht[m,h,:t] @ w[h] used around the MLA attention
// (W_UK absorb and W_UV projection). Replaces XliteOpEinsumMhtHtdMhd / XliteOpEinsumMhtHdtMhd
// (xlite/csrc/op.cpp:1872-1918, kernels/einsum_mht_htd_mhd.h:9-37).
//
// [h,d,t] weights (k-contiguous rows): one wave computes a 32 x 32 output tile with v_mfma_f32_32x32x16,
// operands straight from global memory; a workgroup covers 32 rows x 128 columns.
// [h,t,d] weights (the layout of both mla_v2 einsums): a workgroup covers 32 rows x 64 columns of one head and
// its four waves split the reduction; a wave copies its slab of the weight (rows of 128 contiguous bytes) into
// a region of LDS of its own with 16-byte loads, all of them in flight at once, and reads it back transposed
// (ds_read_b64_tr_b16) as the B operand; the four partial tiles meet through LDS. With m <= 32 (a decode
// step) every weight byte is read once, so the kernel is bound by streaming the weights: many small
// workgroups (h * d / 64) keep every compute unit loading.
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

typedef __attribute__((__vector_size__(4 * sizeof(short)))) short s16x4_t;

constexpr int kSlabCols = 64;                 // output columns of a workgroup
constexpr int kSlabPitch = kSlabCols * 2 + 32;   // LDS bytes of a weight row: 128 + 32 keeps the transposing reads off each other's banks
constexpr int kSlabRowsMax = 64;              // weight rows (k) a wave holds at a time

// A workgroup covers RT row tiles of 32 rows (1 or 2), so that a decode batch of up to 64 rows reads every weight byte
// once. ONCE: the workgroup's rows are all there are (m <= 32 RT), so every weight byte is used once in the launch and
// is fetched with the non-temporal hint (the W_UV projection of a 32-token decode batch: 12.1 -> 7.4 us; with several
// workgroups per weight slab they share the weight lines through L2 and the loads stay plain).
template <typename T, bool ONCE, int RT>
__global__ void __launch_bounds__(256)
einsum_htd_kernel(const uint16_t *__restrict__ mht, const uint16_t *__restrict__ w, uint16_t *__restrict__ mhd,
                  uint32_t m, uint32_t h, uint32_t t, uint32_t d, uint32_t t_stride)
{
    __shared__ __attribute__((aligned(16))) unsigned char slab[4 * kSlabRowsMax * kSlabPitch];   // 40 KiB
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t col = lane & 31, half = lane >> 5;
    const uint32_t head = blockIdx.z;
    const uint32_t m0 = blockIdx.y * (32 * RT);
    const uint32_t n0 = blockIdx.x * kSlabCols;
    bool row_ok[RT];
    const uint16_t *a_ptr[RT];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        const uint32_t row = m0 + 32 * rt + col;
        row_ok[rt] = row < m;
        a_ptr[rt] = mht + (static_cast<uint64_t>(row_ok[rt] ? row : 0) * h + head) * t_stride;
    }
    const uint16_t *w_head = w + static_cast<uint64_t>(head) * t * d + n0;
    unsigned char *mine = slab + wave * (kSlabRowsMax * kSlabPitch);

    // this wave's share of the reduction: a quarter of t, in multiples of 16
    const uint32_t steps = t / 16, per = ceil_div(steps, 4u);
    const uint32_t k_lo = min(steps, wave * per) * 16, k_hi = min(steps, (wave + 1) * per) * 16;

    f32x16_t acc[RT][2];
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
#pragma unroll
        for (int j = 0; j < 2; j++) {
#pragma unroll
            for (int k = 0; k < 16; k++) {
                acc[rt][j][k] = 0.f;
            }
        }
    }
    // transposing read role: the 16-lane group g serves columns 16 (g % 2) .. + 15 of a 32-column tile and the
    // rows 8 (g / 2) .. + 3 (+ 4 for the second read) of a 16-row step; lane 4 j' + q points at row j', columns 4 q .. + 3
    const uint32_t gi = lane & 15, g = lane >> 4;
    const uint32_t tr_off = (8 * (g >> 1) + (gi >> 2)) * kSlabPitch + (16 * (g & 1) + 4 * (gi & 3)) * 2;
    typedef s16x4_t __attribute__((address_space(3))) * lds_tr_ptr;

    for (uint32_t kb = k_lo; kb < k_hi; kb += kSlabRowsMax) {
        const uint32_t rows = min(static_cast<uint32_t>(kSlabRowsMax), k_hi - kb);
        // the slab: `rows` weight rows of 128 bytes = 8 lanes of 16 bytes; 8 rows per wave-wide load
        uint4 v[kSlabRowsMax / 8];
#pragma unroll
        for (int i = 0; i < kSlabRowsMax / 8; i++) {
            const uint32_t r = min(i * 8 + (lane >> 3), rows - 1);   // rows past the slab re-read its last row
            const uint16_t *src = w_head + static_cast<uint64_t>(kb + r) * d + (lane & 7) * 8;
            if constexpr (ONCE) {
                typedef uint32_t words_t __attribute__((ext_vector_type(4)));
                const words_t wv = __builtin_nontemporal_load(reinterpret_cast<const words_t *>(src));
                v[i] = make_uint4(wv.x, wv.y, wv.z, wv.w);
            } else {
                v[i] = *reinterpret_cast<const uint4 *>(src);
            }
        }
#pragma unroll
        for (int i = 0; i < kSlabRowsMax / 8; i++) {
            const uint32_t r = i * 8 + (lane >> 3);
            if (r < rows) {
                *reinterpret_cast<uint4 *>(mine + r * kSlabPitch + (lane & 7) * 16) = v[i];
            }
        }
        // wave-private region: the LDS counter wait the compiler inserts between the writes and the reads is all
        // the ordering needed
        for (uint32_t k0 = 0; k0 < rows; k0 += 16) {
            uint4 a[RT];
#pragma unroll
            for (int rt = 0; rt < RT; rt++) {
                a[rt] = make_uint4(0, 0, 0, 0);
                if (row_ok[rt]) {
                    a[rt] = *reinterpret_cast<const uint4 *>(a_ptr[rt] + kb + k0 + half * 8);
                }
            }
#pragma unroll
            for (int j = 0; j < 2; j++) {
                unsigned char *src = mine + k0 * kSlabPitch + tr_off + j * 64;
                const uint2 b0 = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)src));
                const uint2 b1 = __builtin_bit_cast(uint2, __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_tr_ptr)(src + 4 * kSlabPitch)));
#pragma unroll
                for (int rt = 0; rt < RT; rt++) {
                    acc[rt][j] = Mma<T>::run(a[rt], make_uint4(b0.x, b0.y, b1.x, b1.y), acc[rt][j]);
                }
            }
        }
    }
    // the four partial tiles meet in LDS (the slabs are done with), one row tile at a time: [wave][32 rows][64 columns] fp32
    float *part = reinterpret_cast<float *>(slab);
#pragma unroll
    for (int rt = 0; rt < RT; rt++) {
        __syncthreads();
#pragma unroll
        for (int j = 0; j < 2; j++) {
#pragma unroll
            for (int k = 0; k < 16; k++) {
                const uint32_t r = (k / 4) * 8 + half * 4 + (k % 4);
                part[(wave * 32 + r) * kSlabCols + j * 32 + col] = acc[rt][j][k];
            }
        }
        __syncthreads();
        // thread = (row, 8 columns): sums the four partials and stores 16 bytes
        const uint32_t r = threadIdx.x >> 3, c8 = (threadIdx.x & 7) * 8;
        if (m0 + 32 * rt + r < m) {
            float sum[8];
#pragma unroll
            for (int i = 0; i < 8; i++) {
                sum[i] = 0.f;
            }
#pragma unroll
            for (int wv = 0; wv < 4; wv++) {
                const float4 x = *reinterpret_cast<const float4 *>(part + (wv * 32 + r) * kSlabCols + c8);
                const float4 y = *reinterpret_cast<const float4 *>(part + (wv * 32 + r) * kSlabCols + c8 + 4);
                sum[0] += x.x; sum[1] += x.y; sum[2] += x.z; sum[3] += x.w;
                sum[4] += y.x; sum[5] += y.y; sum[6] += y.z; sum[7] += y.w;
            }
            uint4 o;
            o.x = T::pack(sum[0], sum[1]);
            o.y = T::pack(sum[2], sum[3]);
            o.z = T::pack(sum[4], sum[5]);
            o.w = T::pack(sum[6], sum[7]);
            *reinterpret_cast<uint4 *>(mhd + (static_cast<uint64_t>(m0 + 32 * rt + r) * h + head) * d + n0 + c8) = o;
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
    if (!w_is_hdt && d % kSlabCols == 0) {
        // [h,t,d] weights: the LDS-transposing kernel
        // (more than 32 rows: two row tiles per workgroup, so a decode batch of up to 64 rows streams the weights once)
        const uint32_t rt = m > 32 ? 2 : 1;
        dim3 g2(d / kSlabCols, ceil_div(m, 32 * rt), h);
        const bool once = m <= 32 * rt;
        auto launch = [&](auto tag) {
            using T = decltype(tag);
            if (rt == 2) {
                if (once) {
                    einsum_htd_kernel<T, true, 2><<<g2, 256, 0, s>>>(a, b, c, m, h, t, d, t_stride);
                } else {
                    einsum_htd_kernel<T, false, 2><<<g2, 256, 0, s>>>(a, b, c, m, h, t, d, t_stride);
                }
            } else {
                einsum_htd_kernel<T, true, 1><<<g2, 256, 0, s>>>(a, b, c, m, h, t, d, t_stride);
            }
        };
        if (dtype == XLITE_HIP_BF16) {
            launch(BF16{});
        } else {
            launch(FP16{});
        }
        XL_LAUNCH_CHECK();
        return XLITE_HIP_OK;
    }
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
