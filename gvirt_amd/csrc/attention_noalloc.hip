// The attention operator for callers that cannot allocate device memory (code under HIP graph capture,
// tight serving loops, harnesses that forbid it): the split-KV partial results go to a buffer that is part of
// the library's own device image instead of a caller-provided workspace.
#include <mutex>

#include "attention_common.h"

using namespace xlite;

// One copy per GPU the library is loaded on, at that GPU's own address, held until the process ends. In host
// code this name is a stand-in for the symbol, not a device address: only scratch_of_current_device() below
// may mention it, everything else uses the address that function returns.
static __device__ __align__(256) unsigned char scratch[XLITE_HIP_NOALLOC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
std::mutex g_mu;
void *g_scratch_ptr[kMaxDevices] = {};

// the device address of `scratch` on the current device, looked up once per device
int scratch_of_current_device(void **out)
{
    int dev = 0;
    XL_HIP(hipGetDevice(&dev));
    XL_REQUIRE(dev >= 0 && dev < kMaxDevices, "device ordinal out of range");
    std::lock_guard<std::mutex> lock(g_mu);
    if (g_scratch_ptr[dev] == nullptr) {
        void *ptr = nullptr;
        XL_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
        XL_REQUIRE(ptr != nullptr, "hipGetSymbolAddress returned no address for the scratch buffer");
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return XLITE_HIP_OK;
}

}  // namespace

extern "C" size_t xlite_hip_attention_noalloc_scratch_bytes(void) { return XLITE_HIP_NOALLOC_SCRATCH_BYTES; }

extern "C" int xlite_hip_attention_noalloc(void *stream, const void *qkv, const void *k_cache, const void *v_cache,
                                           void *output, const int32_t *query_start_loc, const int32_t *lens,
                                           const int32_t *cached_lens, const int32_t *block_tables,
                                           uint32_t total_tokens, uint32_t n_heads, uint32_t n_kv_heads,
                                           uint32_t head_dim, uint32_t block_size, uint32_t batch,
                                           uint32_t max_num_block, int dtype, int kv_dtype, const float *k_scale,
                                           const float *v_scale)
{
    if (batch == 0 || total_tokens == 0) {
        return XLITE_HIP_OK;
    }
    const size_t need = xlite_hip_attention_workspace_bytes_kv(total_tokens, n_heads, n_kv_heads, head_dim, block_size,
                                                               batch, max_num_block, kv_dtype);
    if (need > XLITE_HIP_NOALLOC_SCRATCH_BYTES) {
        return fail(XLITE_HIP_ENOSPC, __func__,
                    "this shape needs " + std::to_string(need) + " bytes of scratch, the built-in buffer holds " +
                        std::to_string(static_cast<size_t>(XLITE_HIP_NOALLOC_SCRATCH_BYTES)) +
                        ": use xlite_hip_attention with a workspace");
    }
    void *ws = nullptr;
    if (const int rc = scratch_of_current_device(&ws)) {
        return rc;
    }
    // Nothing in the buffer has to start at zero: every kernel writes the counts, meta entries and partial
    // slots it later reads, so the previous call's contents are simply overwritten.
    return xlite_hip_attention(stream, qkv, k_cache, v_cache, output, query_start_loc, lens, cached_lens, block_tables,
                               total_tokens, n_heads, n_kv_heads, head_dim, block_size, batch, max_num_block, dtype,
                               kv_dtype, k_scale, v_scale, ws, XLITE_HIP_NOALLOC_SCRATCH_BYTES);
}
