// Host-only entry points: error state, device probe, KV-tile tuner, attention metadata.
#include <math.h>

#include <algorithm>
#include <atomic>
#include <cstring>
#include <vector>

#include <map>
#include <mutex>
#include <utility>

#include "common.h"

namespace xlite {

static thread_local std::string g_last_error;

void set_error(const std::string &msg) { g_last_error = msg; }

// Dynamic LDS above 64 KiB has to be allowed per kernel function and per device; remember the largest
// request granted for each pair.
int ensure_dynamic_lds(const void *kernel, size_t bytes)
{
    static std::mutex mu;
    static std::map<std::pair<const void *, int>, size_t> granted;
    int dev = 0;
    XL_HIP(hipGetDevice(&dev));
    std::lock_guard<std::mutex> lock(mu);
    size_t &have = granted[std::make_pair(kernel, dev)];
    if (have < bytes) {
        XL_HIP(hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(bytes)));
        have = bytes;
    }
    return XLITE_HIP_OK;
}

int fail(int code, const char *func, const std::string &msg)
{
    g_last_error = std::string(func) + ": " + msg;
    return code;
}

}  // namespace xlite

using namespace xlite;

extern "C" const char *xlite_hip_last_error(void) { return g_last_error.c_str(); }

static std::atomic<unsigned long long *> g_clock_probe{nullptr};
namespace xlite {
unsigned long long *clock_probe() { return g_clock_probe.load(std::memory_order_relaxed); }
}  // namespace xlite
extern "C" int xlite_hip_set_clock_probe(void *device_words)
{
    g_clock_probe.store(static_cast<unsigned long long *>(device_words), std::memory_order_relaxed);
    return XLITE_HIP_OK;
}

extern "C" int xlite_hip_version(void) { return 1; }

extern "C" int xlite_hip_device_info(int device, int *num_cu, int *lds_bytes_per_cu, char *arch,
                                     size_t arch_len)
{
    hipDeviceProp_t prop;
    XL_HIP(hipGetDeviceProperties(&prop, device));
    if (num_cu) {
        *num_cu = prop.multiProcessorCount;
    }
    if (lds_bytes_per_cu) {
        *lds_bytes_per_cu = static_cast<int>(prop.sharedMemPerMultiprocessor);
    }
    if (arch && arch_len) {
        strncpy(arch, prop.gcnArchName, arch_len - 1);
        arch[arch_len - 1] = 0;
    }
    return XLITE_HIP_OK;
}

// ---- KV tile tuner: same integer results as xlite/csrc/auto_tuner.cpp:10-210 -------------
namespace {

constexpr uint32_t kMaxM0 = 128;            // xlite/csrc/kernels/kernel_param.h:33
constexpr uint32_t kSingleBatchMinTile = 1024;  // xlite/csrc/auto_tuner.h:11
constexpr uint32_t kMinTile = 4096;         // xlite/csrc/auto_tuner.h:12
constexpr uint32_t kMaxTile = 8192;         // xlite/csrc/auto_tuner.h:13

// Tasks (query tile x kv head x kv tile) that see at least one key.
uint32_t count_tasks(uint32_t clen, uint32_t qlen, uint32_t group, uint32_t n_kv, uint32_t tile)
{
    uint32_t qtile = kMaxM0 / group;
    if (qtile == 0) {
        qtile = kMaxM0;
    }
    uint32_t qnum = ceil_div(qlen, qtile);
    uint32_t kvnum = ceil_div(clen + qlen, tile);
    uint32_t valid = 0;
    // a (query tile, kv tile) pair is live when the tile starts before the causal end of the
    // query tile; every kv head contributes one task per live pair
    for (uint32_t qi = 0; qi < qnum; qi++) {
        uint32_t qstart = qi * qtile;
        uint32_t qtl = std::min(qtile, qlen - qstart);
        uint32_t causal_end = clen + qstart + qtl;
        for (uint32_t kv = 0; kv < kvnum; kv++) {
            if (causal_end > kv * tile) {
                valid += n_kv;
            }
        }
    }
    return valid;
}

float tile_score(const uint32_t *clens, const uint32_t *qlens, uint32_t batch, uint32_t group,
                 uint32_t n_kv, uint32_t cores, uint32_t tile)
{
    float kv_total = 0.0f;
    int counted = 0;
    uint32_t tasks = 0;
    for (uint32_t i = 0; i < batch; i++) {
        uint32_t kv = clens[i] + qlens[i];
        if (kv == 1) {
            continue;  // padding sequence
        }
        uint32_t rem = kv % tile;
        kv_total += rem == 0 ? 1.0f : static_cast<float>(rem) / static_cast<float>(tile);
        counted++;
        tasks += count_tasks(clens[i], qlens[i], group, n_kv, tile);
    }
    float kv_score = counted == 0 ? 0.0f : kv_total / static_cast<float>(counted);
    uint32_t rem = tasks % cores;
    float task_score = rem == 0 ? 1.0f : static_cast<float>(rem) / static_cast<float>(cores);
    float size_score = static_cast<float>(tile) / static_cast<float>(kMaxTile);
    volatile float a = kv_score * 0.7f;
    volatile float b = task_score * 0.2f;
    volatile float c = size_score * 0.1f;
    volatile float ab = a + b;
    return ab + c;
}

}  // namespace

extern "C" int xlite_hip_get_tile_size_of_cached_kv(const uint32_t *cached_lens,
                                                    const uint32_t *query_lens, uint32_t batch,
                                                    uint32_t head_num_in_group,
                                                    uint32_t n_kv_heads, uint32_t block_size,
                                                    uint32_t aic_num)
{
    XL_REQUIRE(cached_lens && query_lens, "null length array");
    XL_REQUIRE(head_num_in_group > 0 && n_kv_heads > 0 && block_size > 0 && aic_num > 0,
               "zero head/block/core count");
    bool decode = true;
    for (uint32_t i = 0; i < batch; i++) {
        if (query_lens[i] != 1) {
            decode = false;
            break;
        }
    }
    if (!decode) {
        return aic_num == 24 ? 6016 : 8192;
    }
    if (batch == 1) {
        double clen = static_cast<double>(cached_lens[0]);
        uint32_t tasks = static_cast<uint32_t>(std::round(1.5 * std::sqrt(clen / 1024.0) + 3));
        tasks = std::max(1u, std::min(tasks, aic_num));
        uint32_t tile = ceil_div(static_cast<uint32_t>(std::ceil(clen)), tasks);
        tile = ceil_div(tile, block_size) * block_size;
        tile = std::min(tile, kMaxTile);
        tile = std::max(tile, kSingleBatchMinTile);
        return static_cast<int>(tile);
    }
    XL_REQUIRE(batch > 0, "invalid batch: 0");
    float best_score = -1.0f;
    uint32_t best = kMaxTile;
    for (uint32_t tile = kMaxTile; tile >= kMinTile && tile <= kMaxTile; tile -= block_size) {
        float s = tile_score(cached_lens, query_lens, batch, head_num_in_group, n_kv_heads, aic_num,
                             tile);
        if (s > best_score) {
            best_score = s;
            best = tile;
        }
    }
    return static_cast<int>(best);
}

// ---- attention metadata: host part of XRuntime::PrepareAttn (xlite/csrc/runtime.cpp:438-534) ----
extern "C" int xlite_hip_prepare_attn(const uint32_t *lens, const uint32_t *cached_lens,
                                      uint32_t batch, const int32_t *const *block_table_rows,
                                      const uint32_t *row_lens, uint32_t block_size,
                                      int32_t *query_start_loc, int64_t *position,
                                      int32_t *slot_mapping, int32_t *dense_tables,
                                      size_t dense_capacity, uint32_t *max_num_blocks,
                                      uint32_t *batched_tokens, int *is_decode)
{
    XL_REQUIRE(batch > 0, "invalid batchSize: 0");
    XL_REQUIRE(block_size > 0, "block_size must be positive");
    XL_REQUIRE(lens && cached_lens && block_table_rows && row_lens, "null input");
    XL_REQUIRE(query_start_loc && position && slot_mapping && dense_tables, "null output");
    uint32_t start = 0, max_nb = 0;
    bool multi = false;
    std::vector<uint32_t> nblk(batch);
    for (uint32_t i = 0; i < batch; i++) {
        query_start_loc[i] = static_cast<int32_t>(start);
        start += lens[i];
        nblk[i] = ceil_div(lens[i] + cached_lens[i], block_size);
        max_nb = std::max(max_nb, nblk[i]);
        multi = multi || lens[i] != 1;
        XL_REQUIRE(row_lens[i] >= nblk[i], "block table too small (" + std::to_string(row_lens[i]) +
                                               " < " + std::to_string(nblk[i]) + ")");
    }
    XL_REQUIRE(start > 0, "invalid attnMeta batched tokens(0)");
    XL_REQUIRE(static_cast<size_t>(batch) * max_nb <= dense_capacity, "dense table buffer too small");
    uint32_t k = 0;
    for (uint32_t i = 0; i < batch; i++) {
        for (uint32_t j = 0; j < lens[i]; j++) {
            uint64_t pos = static_cast<uint64_t>(cached_lens[i]) + j;
            position[k] = static_cast<int64_t>(pos);
            slot_mapping[k++] = block_table_rows[i][pos / block_size] * static_cast<int32_t>(block_size) +
                                static_cast<int32_t>(pos % block_size);
        }
    }
    std::fill(dense_tables, dense_tables + static_cast<size_t>(batch) * max_nb, 0);
    for (uint32_t i = 0; i < batch; i++) {
        std::copy(block_table_rows[i], block_table_rows[i] + nblk[i],
                  dense_tables + static_cast<size_t>(i) * max_nb);
    }
    if (max_num_blocks) {
        *max_num_blocks = max_nb;
    }
    if (batched_tokens) {
        *batched_tokens = start;
    }
    if (is_decode) {
        *is_decode = multi ? 0 : 1;
    }
    return XLITE_HIP_OK;
}
