// The small operators around the DSA indexer of an MLA layer (xlite/csrc/model.cpp:285-330): LayerNorm of the
// index key, the general form of the interleaved-pair rope (any column offset, in place or to another tensor,
// or straight into a paged cache), and the column-range scaling of the head weights.
#include "common.h"

namespace xlite {

namespace {

// ---------------------------------------------------------------------------------------
// LayerNorm of the first norm_dim columns of every row (xlite/csrc/op.cpp:607-628 with the defaults of the
// binding, xlite/csrc/_C.cpp:1122-1133; golden torch.nn.functional.layer_norm,
// xlite/tests/kernels/layernorm.py:22-23): y = (x - mean) * rsqrt(var + eps) * w + b in fp32, biased variance,
// rounded once. One 64-lane wave per row.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
layernorm_kernel(const uint16_t *__restrict__ in, const uint16_t *__restrict__ w, const uint16_t *__restrict__ b,
                 uint16_t *__restrict__ out, uint32_t num_rows, uint32_t in_stride, uint32_t out_stride, uint32_t dim,
                 float eps)
{
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t waves = blockDim.x / 64;
    for (uint64_t row = static_cast<uint64_t>(blockIdx.x) * waves + (threadIdx.x >> 6); row < num_rows;
         row += static_cast<uint64_t>(gridDim.x) * waves) {
        const uint16_t *x = in + row * in_stride;
        float sum = 0.f;
        for (uint32_t i = lane; i < dim; i += 64) {
            sum += T::to_f32(x[i]);
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            sum += __shfl_xor(sum, o);
        }
        const float mean = sum / static_cast<float>(dim);
        float var = 0.f;
        for (uint32_t i = lane; i < dim; i += 64) {
            const float d = T::to_f32(x[i]) - mean;
            var += d * d;
        }
#pragma unroll
        for (int o = 32; o > 0; o >>= 1) {
            var += __shfl_xor(var, o);
        }
        const float inv = rsqrtf(var / static_cast<float>(dim) + eps);
        // every lane has read its inputs (the reductions above needed them all) before any output is
        // written: in == out is allowed
        for (uint32_t i = lane; i < dim; i += 64) {
            float y = __fmul_rn(T::to_f32(x[i]) - mean, inv);
            y = __fmul_rn(y, T::to_f32(w[i]));
            y = __fadd_rn(y, T::to_f32(b[i]));
            out[row * out_stride + i] = T::from_f32(y);
        }
    }
}

// ---------------------------------------------------------------------------------------
// output[r][offset + i] = input[r][offset + i] * scale for i < count (xlite/csrc/op.cpp:1644-1680), fp32
// product rounded once. Other columns are not touched.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
muls_kernel(const uint16_t *__restrict__ in, uint16_t *__restrict__ out, uint32_t num_rows, uint32_t row_len,
            uint32_t offset, uint32_t count, float scale)
{
    const uint64_t total = static_cast<uint64_t>(num_rows) * count;
    for (uint64_t idx = blockIdx.x * static_cast<uint64_t>(blockDim.x) + threadIdx.x; idx < total;
         idx += static_cast<uint64_t>(gridDim.x) * blockDim.x) {
        const uint64_t at = (idx / count) * row_len + offset + idx % count;
        out[at] = T::from_f32(__fmul_rn(T::to_f32(in[at]), scale));
    }
}

// ---------------------------------------------------------------------------------------
// Interleaved-pair rope in its general form (xlite/csrc/kernels/rope_complex_and_cache.h:12-241): of every
// head's step_dim columns, the rope_dim columns from `offset` are rotated by freqs[position] and leave
// de-interleaved ([re... | im...]); four fp32 products, one add / sub each, one rounding (:165-205).
//  * without a cache: to output[token][head * out_step_dim + out_offset ...]; output may be the input
//    (xlite/csrc/op.cpp:1106-1126);
//  * with a cache (one head): the vdim columns from `offset` - the rotated ones, then the rest unchanged -
//    go to cache[slot / block_size][slot % block_size], and nothing else is written (:216-221,
//    xlite/csrc/op.cpp:1128-1150).
// One wave per (token, head): every lane holds its pairs in registers before the first store, so the
// de-interleaving may overwrite its own input.
// ---------------------------------------------------------------------------------------
constexpr int kMaxPairsPerLane = 4;   // rope_dim <= 512

template <typename T>
__global__ void __launch_bounds__(256)
rope_complex_general_kernel(uint32_t num_tokens, uint32_t n_heads, uint32_t step_dim, uint32_t rope_dim, uint32_t offset,
                            uint32_t vdim, const uint16_t *in, uint16_t *out, uint32_t out_step_dim,
                            uint32_t out_offset, const float *__restrict__ freqs, const int64_t *__restrict__ position,
                            uint32_t block_size, uint16_t *cache, const int32_t *__restrict__ slot_mapping)
{
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t waves = blockDim.x / 64;
    const uint32_t half = rope_dim / 2;
    const uint64_t rows = static_cast<uint64_t>(num_tokens) * n_heads;
    for (uint64_t th = static_cast<uint64_t>(blockIdx.x) * waves + (threadIdx.x >> 6); th < rows;
         th += static_cast<uint64_t>(gridDim.x) * waves) {
        const uint32_t t = static_cast<uint32_t>(th / n_heads);
        const uint16_t *x = in + th * step_dim + offset;
        const float *f = freqs + static_cast<uint64_t>(position[t]) * rope_dim;
        uint16_t re[kMaxPairsPerLane], im[kMaxPairsPerLane];
#pragma unroll
        for (int k = 0; k < kMaxPairsPerLane; k++) {
            const uint32_t j = lane + 64 * k;
            if (j < half) {
                const uint32_t pair = *reinterpret_cast<const uint32_t *>(x + 2 * j);
                const float2 cs = *reinterpret_cast<const float2 *>(f + 2 * j);
                const float xe = T::to_f32(static_cast<uint16_t>(pair & 0xffffu)), xo = T::to_f32(static_cast<uint16_t>(pair >> 16));
                re[k] = T::from_f32(__fsub_rn(__fmul_rn(xe, cs.x), __fmul_rn(xo, cs.y)));
                im[k] = T::from_f32(__fadd_rn(__fmul_rn(xe, cs.y), __fmul_rn(xo, cs.x)));
            }
        }
        uint16_t *dst;
        if (cache != nullptr) {
            const uint32_t slot = static_cast<uint32_t>(slot_mapping[t]);
            dst = cache + (static_cast<uint64_t>(slot / block_size) * block_size + slot % block_size) * vdim;
            for (uint32_t i = rope_dim + lane; i < vdim; i += 64) {
                dst[i] = x[i];
            }
        } else {
            dst = out + th * out_step_dim + out_offset;
        }
#pragma unroll
        for (int k = 0; k < kMaxPairsPerLane; k++) {
            const uint32_t j = lane + 64 * k;
            if (j < half) {
                dst[j] = re[k];
                dst[half + j] = im[k];
            }
        }
    }
}

uint32_t wave_grid(uint64_t rows)
{
    const uint64_t blocks = (rows + 3) / 4;
    return static_cast<uint32_t>(blocks < 1 ? 1 : (blocks > 4096 ? 4096 : blocks));
}

}  // namespace
}  // namespace xlite

using namespace xlite;

extern "C" int xlite_hip_layernorm(void *stream, const void *in, const void *norm, const void *norm_bias, void *out,
                                   uint32_t num_rows, uint32_t in_stride, uint32_t out_stride, uint32_t norm_dim,
                                   float norm_eps, int dtype)
{
    XL_REQUIRE(dtype == XLITE_HIP_BF16 || dtype == XLITE_HIP_FP16, "dtype unsupported!");
    if (num_rows == 0) {
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(in && norm && norm_bias && out, "null tensor");
    XL_REQUIRE(norm_dim > 0 && norm_dim <= in_stride && norm_dim <= out_stride, "norm_dim exceeds the row length");
    const uint32_t grid = wave_grid(num_rows);
    if (dtype == XLITE_HIP_BF16) {
        layernorm_kernel<BF16><<<grid, 256, 0, as_stream(stream)>>>(
            static_cast<const uint16_t *>(in), static_cast<const uint16_t *>(norm), static_cast<const uint16_t *>(norm_bias),
            static_cast<uint16_t *>(out), num_rows, in_stride, out_stride, norm_dim, norm_eps);
    } else {
        layernorm_kernel<FP16><<<grid, 256, 0, as_stream(stream)>>>(
            static_cast<const uint16_t *>(in), static_cast<const uint16_t *>(norm), static_cast<const uint16_t *>(norm_bias),
            static_cast<uint16_t *>(out), num_rows, in_stride, out_stride, norm_dim, norm_eps);
    }
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

extern "C" int xlite_hip_muls(void *stream, const void *input, void *output, uint32_t num_rows, uint32_t row_len,
                              uint32_t calc_offset, uint32_t calc_num, float scale, int dtype)
{
    XL_REQUIRE(dtype == XLITE_HIP_BF16 || dtype == XLITE_HIP_FP16, "dtype unsupported!");
    if (num_rows == 0) {
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(input && output, "null tensor");
    XL_REQUIRE(calc_offset < row_len, "calcOffset >= shape1");
    if (calc_num > row_len - calc_offset) {
        calc_num = row_len - calc_offset;   // as the reference clips it (xlite/csrc/op.cpp:1666-1668)
    }
    XL_REQUIRE(calc_num > 0, "calcNum should be > 0");
    const uint64_t items = static_cast<uint64_t>(num_rows) * calc_num;
    const uint64_t blocks = (items + 255) / 256;
    const uint32_t grid = static_cast<uint32_t>(blocks > 4096 ? 4096 : blocks);
    if (dtype == XLITE_HIP_BF16) {
        muls_kernel<BF16><<<grid, 256, 0, as_stream(stream)>>>(static_cast<const uint16_t *>(input), static_cast<uint16_t *>(output),
                                                              num_rows, row_len, calc_offset, calc_num, scale);
    } else {
        muls_kernel<FP16><<<grid, 256, 0, as_stream(stream)>>>(static_cast<const uint16_t *>(input), static_cast<uint16_t *>(output),
                                                              num_rows, row_len, calc_offset, calc_num, scale);
    }
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

extern "C" int xlite_hip_rope_complex_and_cache(void *stream, uint32_t num_tokens, uint32_t n_local_heads,
                                                uint32_t step_dim, uint32_t rope_dim, uint32_t offset, uint32_t vdim,
                                                const void *input, void *output, uint32_t out_step_dim,
                                                uint32_t out_offset, const float *freqs, const int64_t *position,
                                                uint32_t block_size, void *cache, const int32_t *slot_mapping, int dtype)
{
    XL_REQUIRE(dtype == XLITE_HIP_BF16 || dtype == XLITE_HIP_FP16, "dtype unsupported!");
    if (num_tokens == 0) {
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(input && freqs && position, "null tensor");
    XL_REQUIRE(rope_dim > 0 && rope_dim % 2 == 0 && rope_dim <= 128 * kMaxPairsPerLane, "rope_dim must be even and at most 512");
    XL_REQUIRE(offset % 2 == 0 && step_dim % 2 == 0, "the rotated columns must start at an even element");
    const bool to_cache = block_size != 0 && cache != nullptr && slot_mapping != nullptr;
    if (to_cache) {
        XL_REQUIRE(n_local_heads == 1, "the cache form takes one head");
        XL_REQUIRE(vdim >= rope_dim && offset + vdim <= step_dim, "vdim must cover the rotated columns inside the row");
    } else {
        XL_REQUIRE(output != nullptr, "output required without a cache");
        XL_REQUIRE(offset + rope_dim <= step_dim && out_offset + rope_dim <= out_step_dim, "rotated columns exceed the row");
        XL_REQUIRE(out_offset % 2 == 0 && out_step_dim % 2 == 0, "the output columns must start at an even element");
    }
    const uint32_t grid = wave_grid(static_cast<uint64_t>(num_tokens) * n_local_heads);
    auto launch = [&](auto tag) {
        using T = decltype(tag);
        rope_complex_general_kernel<T><<<grid, 256, 0, as_stream(stream)>>>(
            num_tokens, n_local_heads, step_dim, rope_dim, offset, vdim, static_cast<const uint16_t *>(input),
            static_cast<uint16_t *>(output), out_step_dim, out_offset, freqs, position, to_cache ? block_size : 0,
            to_cache ? static_cast<uint16_t *>(cache) : nullptr, slot_mapping);
    };
    if (dtype == XLITE_HIP_BF16) {
        launch(BF16{});
    } else {
        launch(FP16{});
    }
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}
