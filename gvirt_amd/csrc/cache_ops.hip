// Paged KV-cache writers and gathers: rope_and_cache, gather_sparse_kv_cache, rope_complex,
// mla_prepare, int8 quantisation. All are HBM-bound copy/elementwise kernels: every thread
// moves 16-byte vectors, adjacent lanes touch adjacent addresses.
#include "rope_item.h"

namespace xlite {

// ---------------------------------------------------------------------------------------
// rope_and_cache (xlite/csrc/kernels/rope_and_cache.h:206-610)
// One item = one (token, head slot, chunk pair): a thread rotates 8 elements of the first
// half of the rotary span together with their 8 partners in the second half (both are
// written in place, so one thread must own both), or copies/scales one pass-through chunk.
// Rounding follows calc_cossin_cast (:93-129): each product is rounded to the storage
// type, the difference/sum is formed in fp32 and rounded again; q is then scaled in fp32
// and rounded once more (:576-586).
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
rope_and_cache_kernel(const RopeArgs r)
{
    const uint32_t items_per_token = rope_items_per_token(r);
    const uint64_t total = static_cast<uint64_t>(r.num_tokens) * items_per_token;
    for (uint64_t idx = blockIdx.x * static_cast<uint64_t>(blockDim.x) + threadIdx.x; idx < total;
         idx += static_cast<uint64_t>(gridDim.x) * blockDim.x) {
        rope_item<T>(r, static_cast<uint32_t>(idx / items_per_token), static_cast<uint32_t>(idx % items_per_token));
    }
}

// ---------------------------------------------------------------------------------------
// gather_sparse_kv_cache (xlite/csrc/kernels/gather_sparse_kv_cache.h:59-125): pure copy.
// One 16-lane group moves the latent row, the rope row follows with the leading lanes.
// ---------------------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
gather_sparse_kernel(const uint4 *__restrict__ k_cache, const uint4 *__restrict__ pe_cache,
                     const int32_t *__restrict__ block_tables, const int32_t *__restrict__ topk,
                     const int32_t *__restrict__ query_lens, const int32_t *__restrict__ cached_lens,
                     uint4 *__restrict__ k_dense, uint4 *__restrict__ pe_dense, uint32_t batch,
                     uint32_t index_topk, uint32_t block_size, uint32_t max_num_blocks,
                     uint32_t k_vecs, uint32_t pe_vecs)
{
    const uint32_t b = blockIdx.y;
    const int32_t total = query_lens[b] + cached_lens[b];
    const uint32_t valid = total <= 0 ? 0u : (static_cast<uint32_t>(total) < index_topk ? total : index_topk);
    const uint32_t group = threadIdx.x / 16, lane = threadIdx.x % 16;
    const uint32_t groups = blockDim.x / 16;
    for (uint32_t i = blockIdx.x * groups + group; i < valid; i += gridDim.x * groups) {
        const uint32_t tok = static_cast<uint32_t>(topk[static_cast<uint64_t>(b) * index_topk + i]);
        const uint32_t phys = static_cast<uint32_t>(block_tables[static_cast<uint64_t>(b) * max_num_blocks + tok / block_size]);
        const uint64_t src = static_cast<uint64_t>(phys) * block_size + tok % block_size;
        const uint64_t dst = static_cast<uint64_t>(b) * index_topk + i;
        for (uint32_t c = lane; c < k_vecs; c += 16) {
            k_dense[dst * k_vecs + c] = k_cache[src * k_vecs + c];
        }
        for (uint32_t c = lane; c < pe_vecs; c += 16) {
            pe_dense[dst * pe_vecs + c] = pe_cache[src * pe_vecs + c];
        }
    }
}

// ---------------------------------------------------------------------------------------
// Interleaved-pair rotation (xlite/csrc/kernels/rope_complex_and_cache.h:165-221): four fp32
// products, one fp32 add/sub each (no fused multiply-add, the reference rounds every
// product), then one rounding to the storage type. A thread produces one (re, im) pair.
// ---------------------------------------------------------------------------------------
template <typename T>
__device__ __forceinline__ void rotate_pair(uint16_t xe_h, uint16_t xo_h, float c, float s,
                                            uint16_t &re, uint16_t &im)
{
    const float xe = T::to_f32(xe_h), xo = T::to_f32(xo_h);
    const float ec = __fmul_rn(xe, c), os = __fmul_rn(xo, s);
    const float es = __fmul_rn(xe, s), oc = __fmul_rn(xo, c);
    re = T::from_f32(__fsub_rn(ec, os));
    im = T::from_f32(__fadd_rn(es, oc));
}

template <typename T>
__global__ void __launch_bounds__(256)
rope_complex_kernel(uint32_t num_tokens, uint32_t n_heads, uint32_t step_dim, uint32_t rope_dim,
                    const uint16_t *__restrict__ input, const float *__restrict__ freqs,
                    const int64_t *__restrict__ position, uint16_t *__restrict__ output)
{
    const uint32_t half = rope_dim / 2;
    const uint64_t total = static_cast<uint64_t>(num_tokens) * n_heads * half;
    for (uint64_t idx = blockIdx.x * static_cast<uint64_t>(blockDim.x) + threadIdx.x; idx < total;
         idx += static_cast<uint64_t>(gridDim.x) * blockDim.x) {
        const uint32_t j = static_cast<uint32_t>(idx % half);
        const uint64_t th = idx / half;  // token * n_heads + head
        const uint32_t t = static_cast<uint32_t>(th / n_heads);
        const uint16_t *x = input + th * step_dim + (step_dim - rope_dim);
        const float2 f = *reinterpret_cast<const float2 *>(freqs + static_cast<uint64_t>(position[t]) * rope_dim + 2 * j);
        const uint32_t pair = *reinterpret_cast<const uint32_t *>(x + 2 * j);
        uint16_t re, im;
        rotate_pair<T>(static_cast<uint16_t>(pair & 0xffffu), static_cast<uint16_t>(pair >> 16), f.x, f.y, re, im);
        output[th * rope_dim + j] = re;
        output[th * rope_dim + half + j] = im;
    }
}

// ---------------------------------------------------------------------------------------
// mla_prepare (xlite/csrc/kernels/mla_prepare.h:14-39): one workgroup per token.
//   phase 1  attn_norm_qc  = rms(q_lora)  * w_q  + b_q
//   phase 2  attn_norm_kvc = rms(kv_lora) * w_kv + b_kv, also stored to k_cache[slot]
//   phase 3  rope slice rotated in place and stored to pe_cache[slot]
// RMSNorm in fp32: x * rsqrt(mean(x^2) + eps) * w + b (xlite/tests/kernels/mla_prepare.py:38-45).
// ---------------------------------------------------------------------------------------
template <typename T>
__device__ float block_sum_sq(const uint16_t *x, uint32_t n, float *red)
{
    float acc = 0.f;
    for (uint32_t i = threadIdx.x; i < n; i += blockDim.x) {
        const float v = T::to_f32(x[i]);
        acc += v * v;
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
        acc += __shfl_xor(acc, o);
    }
    __syncthreads();  // protect `red` against the previous use
    if ((threadIdx.x & 63) == 0) {
        red[threadIdx.x >> 6] = acc;
    }
    __syncthreads();
    float total = 0.f;
    for (uint32_t w = 0; w < blockDim.x / 64; w++) {
        total += red[w];
    }
    return total;
}

template <typename T>
__global__ void __launch_bounds__(256)
mla_prepare_kernel(uint16_t *__restrict__ qkvc, const uint16_t *__restrict__ q_w,
                   const uint16_t *__restrict__ q_b, uint16_t *__restrict__ out_qc,
                   const uint16_t *__restrict__ kv_w, const uint16_t *__restrict__ kv_b,
                   uint16_t *__restrict__ out_kvc, const float *__restrict__ freqs,
                   const int64_t *__restrict__ position, uint16_t *__restrict__ k_cache,
                   uint16_t *__restrict__ pe_cache, const int32_t *__restrict__ slot_mapping,
                   uint32_t q_rank, uint32_t kv_rank, uint32_t rope_dim, uint32_t block_size,
                   float eps)
{
    __shared__ float red[4];
    const uint32_t t = blockIdx.x;
    uint16_t *row = qkvc + static_cast<uint64_t>(t) * (q_rank + kv_rank + rope_dim);
    uint64_t slot_row = 0;
    if (block_size) {
        const uint32_t slot = static_cast<uint32_t>(slot_mapping[t]);
        slot_row = static_cast<uint64_t>(slot / block_size) * block_size + slot % block_size;
    }

    const float ssq_q = block_sum_sq<T>(row, q_rank, red);
    const float inv_q = rsqrtf(ssq_q / static_cast<float>(q_rank) + eps);
    for (uint32_t i = threadIdx.x; i < q_rank; i += blockDim.x) {
        const float y = __fmul_rn(T::to_f32(row[i]), inv_q);
        out_qc[static_cast<uint64_t>(t) * q_rank + i] =
            T::from_f32(__fadd_rn(__fmul_rn(T::to_f32(q_w[i]), y), T::to_f32(q_b[i])));
    }

    const float ssq_kv = block_sum_sq<T>(row + q_rank, kv_rank, red);
    const float inv_kv = rsqrtf(ssq_kv / static_cast<float>(kv_rank) + eps);
    for (uint32_t i = threadIdx.x; i < kv_rank; i += blockDim.x) {
        const float y = __fmul_rn(T::to_f32(row[q_rank + i]), inv_kv);
        const uint16_t o = T::from_f32(__fadd_rn(__fmul_rn(T::to_f32(kv_w[i]), y), T::to_f32(kv_b[i])));
        out_kvc[static_cast<uint64_t>(t) * kv_rank + i] = o;
        if (block_size) {
            k_cache[slot_row * kv_rank + i] = o;
        }
    }

    uint16_t *pe = row + q_rank + kv_rank;
    const uint32_t half = rope_dim / 2;
    const float *f = freqs + static_cast<uint64_t>(position[t]) * rope_dim;
    // every thread reads its pair before anybody writes: the output is de-interleaved, so
    // element j and half + j are written by the thread that read elements 2j and 2j + 1
    uint16_t re = 0, im = 0;
    const bool active = threadIdx.x < half;
    if (active) {
        const uint32_t j = threadIdx.x;
        rotate_pair<T>(pe[2 * j], pe[2 * j + 1], f[2 * j], f[2 * j + 1], re, im);
    }
    __syncthreads();
    if (active) {
        const uint32_t j = threadIdx.x;
        pe[j] = re;
        pe[half + j] = im;
        if (block_size) {
            pe_cache[slot_row * rope_dim + j] = re;
            pe_cache[slot_row * rope_dim + half + j] = im;
        }
    }
}

// ---------------------------------------------------------------------------------------
// int8 KV quantisation: one 16-lane group per row of head_dim elements (head_dim % 8 == 0,
// head_dim <= 128*... handled by a strided loop). scale = absmax / 127.
// ---------------------------------------------------------------------------------------
// ---------------------------------------------------------------------------------------
// qk_rms_norm (xlite/csrc/kernels/qk_rms_norm.h:32-54, arithmetic of xlite/csrc/kernels/norm.h:272-320):
// RMSNorm of the Q segment (q_cnt vectors of q_dim elements from column 0) and of the K segment (k_cnt
// vectors of k_dim elements from column k_start) of every row; other columns are not touched. One 16-lane
// group per vector: y = x * rsqrt(mean(x^2) + eps) * w + b in fp32, rounded once.
// ---------------------------------------------------------------------------------------
template <typename T>
__global__ void __launch_bounds__(256)
qk_rms_norm_kernel(const uint16_t *__restrict__ in, uint16_t *__restrict__ out, const uint16_t *__restrict__ q_w,
                   const uint16_t *__restrict__ q_b, const uint16_t *__restrict__ k_w,
                   const uint16_t *__restrict__ k_b, uint32_t num_tokens, uint32_t row_elems, uint32_t q_dim,
                   uint32_t q_cnt, uint32_t k_dim, uint32_t k_cnt, uint32_t k_start, float eps)
{
    const uint32_t group = threadIdx.x / 16, lane = threadIdx.x % 16;
    const uint32_t groups = blockDim.x / 16;
    const uint32_t per_token = q_cnt + k_cnt;
    const uint64_t vectors = static_cast<uint64_t>(num_tokens) * per_token;
    for (uint64_t v = blockIdx.x * static_cast<uint64_t>(groups) + group; v < vectors;
         v += static_cast<uint64_t>(gridDim.x) * groups) {
        const uint32_t t = static_cast<uint32_t>(v / per_token);
        const uint32_t j = static_cast<uint32_t>(v % per_token);
        const bool is_k = j >= q_cnt;
        const uint32_t dim = is_k ? k_dim : q_dim;
        const uint64_t off = static_cast<uint64_t>(t) * row_elems + (is_k ? k_start + (j - q_cnt) * k_dim : j * q_dim);
        const uint16_t *w = is_k ? k_w : q_w, *b = is_k ? k_b : q_b;
        const uint16_t *x = in + off;
        float acc = 0.f;
        for (uint32_t i = lane; i < dim; i += 16) {
            const float xv = T::to_f32(x[i]);
            acc += xv * xv;
        }
#pragma unroll
        for (int o = 8; o > 0; o >>= 1) {
            acc += __shfl_xor(acc, o);
        }
        const float inv = rsqrtf(acc / static_cast<float>(dim) + eps);
        for (uint32_t i = lane; i < dim; i += 16) {
            float y = __fmul_rn(T::to_f32(x[i]), inv);
            y = __fmul_rn(T::to_f32(w[i]), y);
            if (b != nullptr) {
                y = __fadd_rn(y, T::to_f32(b[i]));
            }
            out[off + i] = T::from_f32(y);
        }
    }
}

// ---------------------------------------------------------------------------------------
// Quantised KV caches (no counterpart in the reference): one fp32 scale per (token, kv head) row,
//   int8:      scale = absmax / 127, q = clamp(rint(x / scale), -127, 127)
//   fp8 e4m3:  scale = absmax / 448, q = e4m3(x / scale) (round to nearest even; 448 is the format's maximum)
// and x^ = q * scale. A row of zeros has scale 0 and is divided by 1 instead.
// ---------------------------------------------------------------------------------------
template <int KV>
struct QuantFmt;
template <>
struct QuantFmt<XLITE_HIP_KV_INT8> {
    static constexpr float kMax = 127.0f;
    // eight quotients -> eight bytes
    static __device__ __forceinline__ uint2 pack8(const float (&y)[8])
    {
        uint32_t w[2] = {0, 0};
#pragma unroll
        for (int j = 0; j < 8; j++) {
            const float q = fminf(fmaxf(rintf(y[j]), -127.f), 127.f);
            w[j / 4] |= (static_cast<uint32_t>(static_cast<int32_t>(q)) & 0xffu) << (8 * (j % 4));
        }
        return make_uint2(w[0], w[1]);
    }
};
template <>
struct QuantFmt<XLITE_HIP_KV_FP8> {
    static constexpr float kMax = 448.0f;
    static __device__ __forceinline__ uint2 pack8(const float (&y)[8])
    {
        int w0 = 0, w1 = 0;
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[0], y[1], w0, false);
        w0 = __builtin_amdgcn_cvt_pk_fp8_f32(y[2], y[3], w0, true);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[4], y[5], w1, false);
        w1 = __builtin_amdgcn_cvt_pk_fp8_f32(y[6], y[7], w1, true);
        return make_uint2(static_cast<uint32_t>(w0), static_cast<uint32_t>(w1));
    }
};

template <typename T>
__device__ __forceinline__ float chunk_absmax(const Vec16 &a)
{
    float m = 0.f;
#pragma unroll
    for (int j = 0; j < 8; j++) {
        m = fmaxf(m, fabsf(T::to_f32(a.h[j])));
    }
    return m;
}

template <typename T, int KV>
__device__ __forceinline__ uint2 quantize_chunk(const Vec16 &a, float safe)
{
    float y[8];
#pragma unroll
    for (int j = 0; j < 8; j++) {
        y[j] = T::to_f32(a.h[j]) / safe;
    }
    return QuantFmt<KV>::pack8(y);
}

// max over the 16 lanes of a group
__device__ __forceinline__ float group16_max(float m)
{
#pragma unroll
    for (int o = 8; o > 0; o >>= 1) {
        m = fmaxf(m, __shfl_xor(m, o));
    }
    return m;
}

// one row (head_dim a multiple of 8) by the 16 lanes of a group, a 16-byte chunk per lane and turn
template <typename T, int KV>
__device__ __forceinline__ void quantize_row(const uint16_t *x, unsigned char *dst, float *scale_out, uint32_t head_dim,
                                             uint32_t lane)
{
    float amax = 0.f;
    for (uint32_t c = lane; c < head_dim / 8; c += 16) {
        Vec16 a;
        a.v = *reinterpret_cast<const uint4 *>(x + c * 8);
        amax = fmaxf(amax, chunk_absmax<T>(a));
    }
    amax = group16_max(amax);
    const float scale = amax / QuantFmt<KV>::kMax;
    const float safe = scale > 0.f ? scale : 1.0f;
    for (uint32_t c = lane; c < head_dim / 8; c += 16) {
        Vec16 a;
        a.v = *reinterpret_cast<const uint4 *>(x + c * 8);
        *reinterpret_cast<uint2 *>(dst + c * 8) = quantize_chunk<T, KV>(a, safe);
    }
    if (lane == 0) {
        *scale_out = scale;
    }
}

template <typename T, int KV>
__global__ void __launch_bounds__(256)
quantize_kv_kernel(const uint16_t *__restrict__ src, unsigned char *__restrict__ dst,
                   float *__restrict__ scales, uint64_t rows, uint32_t head_dim)
{
    const uint32_t group = threadIdx.x / 16, lane = threadIdx.x % 16;
    const uint32_t groups = blockDim.x / 16;
    for (uint64_t r = blockIdx.x * static_cast<uint64_t>(groups) + group; r < rows;
         r += static_cast<uint64_t>(gridDim.x) * groups) {
        quantize_row<T, KV>(src + r * head_dim, dst + r * head_dim, scales + r, head_dim, lane);
    }
}

// The K (already rotated) and V rows of the fused activation rows, quantised into the caches at the
// tokens' slots: row r = (token, K | V, kv head). The second launch of the two-launch form, for head shapes the
// fused kernel below does not take.
template <typename T, int KV>
__global__ void __launch_bounds__(256)
quantize_to_cache_kernel(const uint16_t *__restrict__ inout, unsigned char *__restrict__ k_cache,
                         unsigned char *__restrict__ v_cache, float *__restrict__ k_scale, float *__restrict__ v_scale,
                         const int32_t *__restrict__ slot_mapping, uint32_t num_tokens, uint32_t n_heads,
                         uint32_t n_kv_heads, uint32_t head_dim)
{
    const uint32_t group = threadIdx.x / 16, lane = threadIdx.x % 16;
    const uint32_t groups = blockDim.x / 16;
    const uint64_t rows = static_cast<uint64_t>(num_tokens) * 2 * n_kv_heads;
    const uint32_t slots = n_heads + 2 * n_kv_heads;
    for (uint64_t r = blockIdx.x * static_cast<uint64_t>(groups) + group; r < rows;
         r += static_cast<uint64_t>(gridDim.x) * groups) {
        const uint32_t t = static_cast<uint32_t>(r / (2 * n_kv_heads));
        const uint32_t rem = static_cast<uint32_t>(r % (2 * n_kv_heads));
        const bool is_v = rem >= n_kv_heads;
        const uint32_t kvh = is_v ? rem - n_kv_heads : rem;
        const uint16_t *x = inout + (static_cast<uint64_t>(t) * slots + n_heads + rem) * head_dim;
        const uint64_t row = static_cast<uint64_t>(static_cast<uint32_t>(slot_mapping[t])) * n_kv_heads + kvh;
        quantize_row<T, KV>(x, (is_v ? v_cache : k_cache) + row * head_dim, (is_v ? v_scale : k_scale) + row, head_dim, lane);
    }
}

// rope_and_cache with the quantisation fused into the write (one launch): a group of 16 lanes owns one
// (token, head slot), a lane one item of it - a chunk pair of the rotary span or a chunk beyond it - so heads
// of at most 16 items (head_dim 128 with any rotary span, head_dim 256 fully rotated). q heads are rotated and
// scaled in place; k heads are rotated in place, v heads left as they are, and both go to the cache as the
// quantisation of the 16-bit row: the group's lanes agree on the row's absmax by four exchanges.
template <typename T, int KV>
__global__ void __launch_bounds__(256)
rope_quant_cache_kernel(uint16_t *__restrict__ inout, unsigned char *__restrict__ k_cache,
                        unsigned char *__restrict__ v_cache, float *__restrict__ k_scale, float *__restrict__ v_scale,
                        const int64_t *__restrict__ position, const uint16_t *__restrict__ cosin,
                        const int32_t *__restrict__ slot_mapping, uint32_t num_tokens, uint32_t n_heads,
                        uint32_t n_kv_heads, uint32_t head_dim, uint32_t rot_dim, float q_scale, uint64_t mask_h,
                        uint64_t mask_w)
{
    const uint32_t rot_pairs = rot_dim / 16;
    const uint32_t items_per_head = head_dim / 8 - rot_pairs;   // <= 16
    const uint32_t slots = n_heads + 2 * n_kv_heads;
    const uint32_t half = rot_dim / 2;
    const uint32_t group = threadIdx.x / 16, lane = threadIdx.x % 16;
    const uint32_t groups = blockDim.x / 16;
    const uint64_t total = static_cast<uint64_t>(num_tokens) * slots;
    // every lane of a group runs the same number of turns: the exchanges below need all sixteen
    for (uint64_t g = blockIdx.x * static_cast<uint64_t>(groups) + group; g < total;
         g += static_cast<uint64_t>(gridDim.x) * groups) {
        const uint32_t t = static_cast<uint32_t>(g / slots);
        const uint32_t hs = static_cast<uint32_t>(g % slots);
        uint16_t *row = inout + (static_cast<uint64_t>(t) * slots + hs) * head_dim;
        const bool is_q = hs < n_heads;
        const bool is_k = !is_q && hs < n_heads + n_kv_heads;
        const bool active = lane < items_per_head;
        const bool rot = active && lane < rot_pairs;
        const uint32_t e0 = rot ? lane * 8 : (lane + rot_pairs) * 8;
        const int64_t pos_t = position[t];   // requested with the row, not behind it
        Vec16 a, b;
        a.v = make_uint4(0, 0, 0, 0);
        b.v = make_uint4(0, 0, 0, 0);
        if (active) {
            a.v = *reinterpret_cast<const uint4 *>(row + e0);
            if (rot) {
                b.v = *reinterpret_cast<const uint4 *>(row + e0 + half);
            }
            if (rot && (is_q || is_k)) {
                rotate_chunk_pair<T>(a, b, e0, half, t, pos_t, num_tokens, rot_dim, position, cosin, mask_h, mask_w, is_q, q_scale);
                *reinterpret_cast<uint4 *>(row + e0) = a.v;
                *reinterpret_cast<uint4 *>(row + e0 + half) = b.v;
            } else if (is_q) {
#pragma unroll
                for (int j = 0; j < 8; j++) {
                    a.h[j] = T::from_f32(T::to_f32(a.h[j]) * q_scale);
                }
                *reinterpret_cast<uint4 *>(row + e0) = a.v;
            }
        }
        if (is_q) {
            continue;   // uniform inside the group
        }
        const float amax = group16_max(fmaxf(chunk_absmax<T>(a), chunk_absmax<T>(b)));
        const float scale = amax / QuantFmt<KV>::kMax;
        const float safe = scale > 0.f ? scale : 1.0f;
        const uint32_t kvh = is_k ? hs - n_heads : hs - n_heads - n_kv_heads;
        const uint64_t crow = static_cast<uint64_t>(static_cast<uint32_t>(slot_mapping[t])) * n_kv_heads + kvh;
        unsigned char *dst = (is_k ? k_cache : v_cache) + crow * head_dim;
        if (active) {
            *reinterpret_cast<uint2 *>(dst + e0) = quantize_chunk<T, KV>(a, safe);
            if (rot) {
                *reinterpret_cast<uint2 *>(dst + e0 + half) = quantize_chunk<T, KV>(b, safe);
            }
        }
        if (lane == 0) {
            (is_k ? k_scale : v_scale)[crow] = scale;
        }
    }
}

static uint32_t grid_for(uint64_t work_threads, uint32_t block)
{
    uint64_t blocks = (work_threads + block - 1) / block;
    const uint64_t cap = 256ull * 16;  // 16 workgroups per compute unit is plenty for a copy
    return static_cast<uint32_t>(blocks < 1 ? 1 : (blocks > cap ? cap : blocks));
}

}  // namespace xlite

using namespace xlite;

// Argument checks shared by the rope launchers; *q_scale receives the factor applied to q.
static int rope_check(const void *inout, const int64_t *position, const void *cosin, const int32_t *slot_mapping,
                      uint32_t num_tokens, uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim, uint32_t rot_dim,
                      uint32_t block_size, int is_neox, uint64_t mrope_mask_h, uint64_t mrope_mask_w, int dtype,
                      float *q_scale)
{
    XL_REQUIRE(is_neox, "unsupported rope type gptj");
    XL_REQUIRE(dtype == XLITE_HIP_FP16 || dtype == XLITE_HIP_BF16, "dtype unsupported!");
    if (num_tokens == 0) {
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(inout && position && cosin && slot_mapping, "null tensor");
    XL_REQUIRE(n_heads > 0 && n_kv_heads > 0 && block_size > 0, "zero head count or block size");
    XL_REQUIRE(head_dim % 8 == 0 && head_dim > 0, "head_dim must be a multiple of 8");
    XL_REQUIRE(rot_dim % 16 == 0 && rot_dim > 0 && rot_dim <= head_dim,
               "rot_dim must be a multiple of 16 and at most head_dim");
    XL_REQUIRE(((mrope_mask_h | mrope_mask_w) == 0) || rot_dim <= 128,
               "mrope masks address at most 64 rotary lanes");
    XL_REQUIRE((mrope_mask_h & mrope_mask_w) == 0, "mrope masks must be disjoint");
    float scale = 1.0f / sqrtf(static_cast<float>(head_dim));
    if (dtype == XLITE_HIP_FP16) {
        // the fp16 kernel of the reference multiplies by the scale rounded to fp16
        scale = static_cast<float>(static_cast<_Float16>(scale));
    }
    *q_scale = scale;
    return XLITE_HIP_OK;
}

// Checks the arguments of a rope_and_cache call and gathers them for the kernels (`with_cache` false: the 16-bit caches
// are not written).
int xlite::rope_prepare(void *inout, void *k_cache, void *v_cache, const int64_t *position, const void *cosin,
                        const int32_t *slot_mapping, uint32_t num_tokens, uint32_t n_heads, uint32_t n_kv_heads,
                        uint32_t head_dim, uint32_t rot_dim, uint32_t block_size, int is_neox, uint64_t mrope_mask_h,
                        uint64_t mrope_mask_w, int dtype, bool with_cache, RopeArgs *out)
{
    float scale = 0.f;
    if (const int rc = rope_check(inout, position, cosin, slot_mapping, num_tokens, n_heads, n_kv_heads, head_dim, rot_dim,
                                  block_size, is_neox, mrope_mask_h, mrope_mask_w, dtype, &scale)) {
        return rc;
    }
    XL_REQUIRE(num_tokens == 0 || !with_cache || (k_cache && v_cache), "null tensor");
    RopeArgs r{};
    r.inout = static_cast<uint16_t *>(inout);
    r.k_cache = with_cache ? static_cast<uint16_t *>(k_cache) : nullptr;
    r.v_cache = with_cache ? static_cast<uint16_t *>(v_cache) : nullptr;
    r.position = position;
    r.cosin = static_cast<const uint16_t *>(cosin);
    r.slot_mapping = slot_mapping;
    r.num_tokens = num_tokens;
    r.n_heads = n_heads;
    r.n_kv_heads = n_kv_heads;
    r.head_dim = head_dim;
    r.rot_dim = rot_dim;
    r.block_size = block_size;
    r.q_scale = scale;
    r.mask_h = mrope_mask_h;
    r.mask_w = mrope_mask_w;
    *out = r;
    return XLITE_HIP_OK;
}

// Launch of the rope kernel; with `with_cache` false the 16-bit caches are not written.
static int rope_launch(void *stream, void *inout, void *k_cache, void *v_cache, const int64_t *position,
                       const void *cosin, const int32_t *slot_mapping, uint32_t num_tokens, uint32_t n_heads,
                       uint32_t n_kv_heads, uint32_t head_dim, uint32_t rot_dim, uint32_t block_size, int is_neox,
                       uint64_t mrope_mask_h, uint64_t mrope_mask_w, int dtype, bool with_cache)
{
    RopeArgs r{};
    if (const int rc = rope_prepare(inout, k_cache, v_cache, position, cosin, slot_mapping, num_tokens, n_heads, n_kv_heads,
                                    head_dim, rot_dim, block_size, is_neox, mrope_mask_h, mrope_mask_w, dtype, with_cache,
                                    &r)) {
        return rc;
    }
    if (num_tokens == 0) {
        return XLITE_HIP_OK;
    }
    const uint64_t items = static_cast<uint64_t>(num_tokens) * (n_heads + 2 * n_kv_heads) *
                           (head_dim / 8 - rot_dim / 16);
    const uint32_t grid = grid_for(items, 256);
    auto launch = [&](auto tag) {
        using T = decltype(tag);
        rope_and_cache_kernel<T><<<grid, 256, 0, as_stream(stream)>>>(r);
    };
    if (dtype == XLITE_HIP_BF16) {
        launch(BF16{});
    } else {
        launch(FP16{});
    }
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

extern "C" int xlite_hip_rope_and_cache(void *stream, void *inout, void *k_cache, void *v_cache,
                                        const int64_t *position, const void *cosin,
                                        const int32_t *slot_mapping, uint32_t num_tokens,
                                        uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                                        uint32_t rot_dim, uint32_t block_size, int is_neox,
                                        uint64_t mrope_mask_h, uint64_t mrope_mask_w, int dtype)
{
    return rope_launch(stream, inout, k_cache, v_cache, position, cosin, slot_mapping, num_tokens, n_heads, n_kv_heads,
                       head_dim, rot_dim, block_size, is_neox, mrope_mask_h, mrope_mask_w, dtype, true);
}

extern "C" int xlite_hip_rope_and_cache_quant(void *stream, void *inout, void *k_cache, void *v_cache,
                                              float *k_scale, float *v_scale, const int64_t *position,
                                              const void *cosin, const int32_t *slot_mapping, uint32_t num_tokens,
                                              uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                                              uint32_t rot_dim, uint32_t block_size, int is_neox,
                                              uint64_t mrope_mask_h, uint64_t mrope_mask_w, int dtype, int kv_dtype)
{
    XL_REQUIRE(kv_dtype == XLITE_HIP_KV_INT8 || kv_dtype == XLITE_HIP_KV_FP8, "kv cache dtype unsupported!");
    unsigned char *kc = static_cast<unsigned char *>(k_cache), *vc = static_cast<unsigned char *>(v_cache);
    const bool fused = head_dim % 8 == 0 && rot_dim % 16 == 0 && rot_dim <= head_dim && head_dim / 8 - rot_dim / 16 <= 16;
    if (!fused) {
        // wide heads: the rotation first, then a quantising write of the rotated K rows and the V rows
        const int rc = rope_launch(stream, inout, nullptr, nullptr, position, cosin, slot_mapping, num_tokens, n_heads,
                                   n_kv_heads, head_dim, rot_dim, block_size, is_neox, mrope_mask_h, mrope_mask_w, dtype,
                                   false);
        if (rc != XLITE_HIP_OK || num_tokens == 0) {
            return rc;
        }
        XL_REQUIRE(k_cache && v_cache && k_scale && v_scale, "null tensor");
        const uint32_t grid = grid_for(static_cast<uint64_t>(num_tokens) * 2 * n_kv_heads * 16, 256);
        auto launch = [&](auto tag, auto kv) {
            using T = decltype(tag);
            quantize_to_cache_kernel<T, decltype(kv)::value><<<grid, 256, 0, as_stream(stream)>>>(
                static_cast<const uint16_t *>(inout), kc, vc, k_scale, v_scale, slot_mapping, num_tokens, n_heads, n_kv_heads,
                head_dim);
        };
        using I8 = std::integral_constant<int, XLITE_HIP_KV_INT8>;
        using F8 = std::integral_constant<int, XLITE_HIP_KV_FP8>;
        if (dtype == XLITE_HIP_BF16) {
            kv_dtype == XLITE_HIP_KV_INT8 ? launch(BF16{}, I8{}) : launch(BF16{}, F8{});
        } else {
            kv_dtype == XLITE_HIP_KV_INT8 ? launch(FP16{}, I8{}) : launch(FP16{}, F8{});
        }
        XL_LAUNCH_CHECK();
        return XLITE_HIP_OK;
    }
    float scale = 0.f;
    if (const int rc = rope_check(inout, position, cosin, slot_mapping, num_tokens, n_heads, n_kv_heads, head_dim, rot_dim,
                                  block_size, is_neox, mrope_mask_h, mrope_mask_w, dtype, &scale)) {
        return rc;
    }
    if (num_tokens == 0) {
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(k_cache && v_cache && k_scale && v_scale, "null tensor");
    const uint32_t grid = grid_for(static_cast<uint64_t>(num_tokens) * (n_heads + 2 * n_kv_heads) * 16, 256);
    auto launch = [&](auto tag, auto kv) {
        using T = decltype(tag);
        rope_quant_cache_kernel<T, decltype(kv)::value><<<grid, 256, 0, as_stream(stream)>>>(
            static_cast<uint16_t *>(inout), kc, vc, k_scale, v_scale, position, static_cast<const uint16_t *>(cosin),
            slot_mapping, num_tokens, n_heads, n_kv_heads, head_dim, rot_dim, scale, mrope_mask_h, mrope_mask_w);
    };
    using I8 = std::integral_constant<int, XLITE_HIP_KV_INT8>;
    using F8 = std::integral_constant<int, XLITE_HIP_KV_FP8>;
    if (dtype == XLITE_HIP_BF16) {
        kv_dtype == XLITE_HIP_KV_INT8 ? launch(BF16{}, I8{}) : launch(BF16{}, F8{});
    } else {
        kv_dtype == XLITE_HIP_KV_INT8 ? launch(FP16{}, I8{}) : launch(FP16{}, F8{});
    }
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

extern "C" int xlite_hip_rope_and_cache_int8(void *stream, void *inout, int8_t *k_cache, int8_t *v_cache,
                                             float *k_scale, float *v_scale, const int64_t *position,
                                             const void *cosin, const int32_t *slot_mapping, uint32_t num_tokens,
                                             uint32_t n_heads, uint32_t n_kv_heads, uint32_t head_dim,
                                             uint32_t rot_dim, uint32_t block_size, int is_neox,
                                             uint64_t mrope_mask_h, uint64_t mrope_mask_w, int dtype)
{
    return xlite_hip_rope_and_cache_quant(stream, inout, k_cache, v_cache, k_scale, v_scale, position, cosin, slot_mapping,
                                          num_tokens, n_heads, n_kv_heads, head_dim, rot_dim, block_size, is_neox,
                                          mrope_mask_h, mrope_mask_w, dtype, XLITE_HIP_KV_INT8);
}

extern "C" int xlite_hip_qk_rms_norm(void *stream, const void *in, void *out, const void *q_norm,
                                     const void *q_norm_bias, const void *k_norm, const void *k_norm_bias,
                                     uint32_t num_tokens, uint32_t row_elems, uint32_t q_norm_dim,
                                     uint32_t q_cnt_per_token, uint32_t k_norm_dim, uint32_t k_cnt_per_token,
                                     uint32_t k_start_offset, float norm_eps, int dtype)
{
    XL_REQUIRE(dtype == XLITE_HIP_BF16 || dtype == XLITE_HIP_FP16, "dtype unsupported!");
    if (num_tokens == 0 || q_cnt_per_token + k_cnt_per_token == 0) {
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(in && out, "null tensor");
    XL_REQUIRE(q_cnt_per_token == 0 || (q_norm && q_norm_dim > 0), "Q segment needs a weight and a positive size");
    XL_REQUIRE(k_cnt_per_token == 0 || (k_norm && k_norm_dim > 0), "K segment needs a weight and a positive size");
    XL_REQUIRE(static_cast<uint64_t>(q_norm_dim) * q_cnt_per_token <= k_start_offset || k_cnt_per_token == 0,
               "segments overlap");
    XL_REQUIRE(static_cast<uint64_t>(k_start_offset) + static_cast<uint64_t>(k_norm_dim) * k_cnt_per_token <= row_elems &&
                   static_cast<uint64_t>(q_norm_dim) * q_cnt_per_token <= row_elems,
               "segments exceed the row");
    const uint32_t grid = grid_for(static_cast<uint64_t>(num_tokens) * (q_cnt_per_token + k_cnt_per_token) * 16, 256);
    auto launch = [&](auto tag) {
        using T = decltype(tag);
        qk_rms_norm_kernel<T><<<grid, 256, 0, as_stream(stream)>>>(
            static_cast<const uint16_t *>(in), static_cast<uint16_t *>(out), static_cast<const uint16_t *>(q_norm),
            static_cast<const uint16_t *>(q_norm_bias), static_cast<const uint16_t *>(k_norm),
            static_cast<const uint16_t *>(k_norm_bias), num_tokens, row_elems, q_norm_dim, q_cnt_per_token, k_norm_dim,
            k_cnt_per_token, k_start_offset, norm_eps);
    };
    if (dtype == XLITE_HIP_BF16) {
        launch(BF16{});
    } else {
        launch(FP16{});
    }
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

extern "C" int xlite_hip_gather_sparse_kv_cache(void *stream, const void *k_cache,
                                                const void *pe_cache, const int32_t *block_tables,
                                                const int32_t *topk_indices,
                                                const int32_t *query_lens,
                                                const int32_t *cached_lens, void *k_dense,
                                                void *pe_dense, uint32_t batch, uint32_t index_topk,
                                                uint32_t block_size, uint32_t max_num_blocks,
                                                uint32_t kv_lora_rank, uint32_t rope_head_dim,
                                                uint32_t kv_heads, int dtype)
{
    XL_REQUIRE(kv_heads == 1, "kvHeads should be less than or equal to 1");
    XL_REQUIRE(dtype == XLITE_HIP_BF16 || dtype == XLITE_HIP_FP16, "dtype unsupported!");
    if (batch == 0 || index_topk == 0) {
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(k_cache && pe_cache && block_tables && topk_indices && query_lens && cached_lens &&
                   k_dense && pe_dense,
               "null tensor");
    XL_REQUIRE(kv_lora_rank % 8 == 0 && rope_head_dim % 8 == 0, "row sizes must be multiples of 8");
    XL_REQUIRE(block_size > 0, "block_size must be positive");
    if (batch == 0 || index_topk == 0) {
        return XLITE_HIP_OK;
    }
    dim3 grid(ceil_div(index_topk, 16), batch);
    gather_sparse_kernel<<<grid, 256, 0, as_stream(stream)>>>(
        static_cast<const uint4 *>(k_cache), static_cast<const uint4 *>(pe_cache), block_tables,
        topk_indices, query_lens, cached_lens, static_cast<uint4 *>(k_dense),
        static_cast<uint4 *>(pe_dense), batch, index_topk, block_size, max_num_blocks,
        kv_lora_rank / 8, rope_head_dim / 8);
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

extern "C" int xlite_hip_rope_complex(void *stream, uint32_t num_tokens, uint32_t n_local_heads,
                                      uint32_t step_dim, uint32_t rope_dim, const void *input,
                                      const float *freqs, const int64_t *position, void *output,
                                      int dtype)
{
    XL_REQUIRE(dtype == XLITE_HIP_BF16 || dtype == XLITE_HIP_FP16, "dtype TODO");
    if (num_tokens == 0 || n_local_heads == 0) {
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(input && freqs && position && output, "null tensor");
    XL_REQUIRE(rope_dim % 2 == 0 && rope_dim > 0 && rope_dim <= step_dim, "bad rope_dim");
    XL_REQUIRE(step_dim % 2 == 0, "step_dim must be even");
    if (num_tokens == 0 || n_local_heads == 0) {
        return XLITE_HIP_OK;
    }
    const uint64_t items = static_cast<uint64_t>(num_tokens) * n_local_heads * (rope_dim / 2);
    const uint32_t grid = grid_for(items, 256);
    if (dtype == XLITE_HIP_BF16) {
        rope_complex_kernel<BF16><<<grid, 256, 0, as_stream(stream)>>>(
            num_tokens, n_local_heads, step_dim, rope_dim, static_cast<const uint16_t *>(input), freqs,
            position, static_cast<uint16_t *>(output));
    } else {
        rope_complex_kernel<FP16><<<grid, 256, 0, as_stream(stream)>>>(
            num_tokens, n_local_heads, step_dim, rope_dim, static_cast<const uint16_t *>(input), freqs,
            position, static_cast<uint16_t *>(output));
    }
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

extern "C" int xlite_hip_mla_prepare(void *stream, void *attn_qkvc, const void *q_norm,
                                     const void *q_norm_bias, void *attn_norm_qc,
                                     const void *kv_norm, const void *kv_norm_bias,
                                     void *attn_norm_kvc, const float *freqs,
                                     const int64_t *position, uint32_t num_tokens,
                                     uint32_t q_lora_rank, uint32_t kv_lora_rank,
                                     uint32_t rope_head_dim, uint32_t block_size, void *k_cache,
                                     void *pe_cache, const int32_t *slot_mapping, float norm_eps,
                                     int dtype)
{
    XL_REQUIRE(dtype == XLITE_HIP_BF16 || dtype == XLITE_HIP_FP16, "dtype unsupported!");
    if (num_tokens == 0) {
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(attn_qkvc && q_norm && q_norm_bias && attn_norm_qc && kv_norm && kv_norm_bias &&
                   attn_norm_kvc && freqs && position,
               "null tensor");
    XL_REQUIRE(block_size == 0 || (k_cache && pe_cache && slot_mapping),
               "cache tensors required when block_size != 0");
    XL_REQUIRE(rope_head_dim % 2 == 0 && rope_head_dim > 0 && rope_head_dim <= 512,
               "rope_head_dim must be even and at most 512");
    XL_REQUIRE(q_lora_rank > 0 && kv_lora_rank > 0, "zero rank");
    XL_REQUIRE((q_lora_rank + kv_lora_rank) % 2 == 0, "rope slice must start at an even element");
    if (num_tokens == 0) {
        return XLITE_HIP_OK;
    }
    auto launch = [&](auto tag) {
        using T = decltype(tag);
        mla_prepare_kernel<T><<<num_tokens, 256, 0, as_stream(stream)>>>(
            static_cast<uint16_t *>(attn_qkvc), static_cast<const uint16_t *>(q_norm),
            static_cast<const uint16_t *>(q_norm_bias), static_cast<uint16_t *>(attn_norm_qc),
            static_cast<const uint16_t *>(kv_norm), static_cast<const uint16_t *>(kv_norm_bias),
            static_cast<uint16_t *>(attn_norm_kvc), freqs, position, static_cast<uint16_t *>(k_cache),
            static_cast<uint16_t *>(pe_cache), slot_mapping, q_lora_rank, kv_lora_rank,
            rope_head_dim, block_size, norm_eps);
    };
    if (dtype == XLITE_HIP_BF16) {
        launch(BF16{});
    } else {
        launch(FP16{});
    }
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

extern "C" int xlite_hip_quantize_kv(void *stream, const void *src, void *dst, float *scales, uint64_t rows,
                                     uint32_t head_dim, int dtype, int kv_dtype)
{
    XL_REQUIRE(dtype == XLITE_HIP_BF16 || dtype == XLITE_HIP_FP16, "dtype unsupported!");
    XL_REQUIRE(kv_dtype == XLITE_HIP_KV_INT8 || kv_dtype == XLITE_HIP_KV_FP8, "kv cache dtype unsupported!");
    if (rows == 0) {
        return XLITE_HIP_OK;
    }
    XL_REQUIRE(src && dst && scales, "null tensor");
    XL_REQUIRE(head_dim > 0 && head_dim % 8 == 0, "head_dim must be a positive multiple of 8");
    const uint32_t grid = grid_for(rows * 16, 256);
    auto launch = [&](auto tag, auto kv) {
        using T = decltype(tag);
        quantize_kv_kernel<T, decltype(kv)::value><<<grid, 256, 0, as_stream(stream)>>>(
            static_cast<const uint16_t *>(src), static_cast<unsigned char *>(dst), scales, rows, head_dim);
    };
    using I8 = std::integral_constant<int, XLITE_HIP_KV_INT8>;
    using F8 = std::integral_constant<int, XLITE_HIP_KV_FP8>;
    if (dtype == XLITE_HIP_BF16) {
        kv_dtype == XLITE_HIP_KV_INT8 ? launch(BF16{}, I8{}) : launch(BF16{}, F8{});
    } else {
        kv_dtype == XLITE_HIP_KV_INT8 ? launch(FP16{}, I8{}) : launch(FP16{}, F8{});
    }
    XL_LAUNCH_CHECK();
    return XLITE_HIP_OK;
}

extern "C" int xlite_hip_quantize_kv_int8(void *stream, const void *src, int8_t *dst, float *scales,
                                          uint64_t rows, uint32_t head_dim, int dtype)
{
    return xlite_hip_quantize_kv(stream, src, dst, scales, rows, head_dim, dtype, XLITE_HIP_KV_INT8);
}
