// Measurement aid: how fast this part streams KV pages when nothing is computed on them.  The decode kernels are
// bound by HBM bandwidth; the figure they are held against is what a plain reader reaches over the same pools, with
// the same 16-byte accesses and page-sized pieces, and the same bytes per launch: one launch reads the pages of two
// pools (K and V).  512 workgroups of four waves (two per CU); a wave reads whole pages (a contiguous run of page_bytes,
// or the page a table of ids names), eight 16-byte loads per lane in flight, and folds what it read into one word so
// that the loads cannot be dropped.  With ids, a wave either fetches a run's id when it gets to the run (a dependent
// fetch per run) or one run ahead.

#include "device_common.hpp"

namespace areno {
namespace {

constexpr int kProbeWaves = 4;        // per workgroup
constexpr int kProbeWorkgroups = 512;  // two per CU
constexpr int kProbeLoads = 8;         // 16-byte loads per lane in flight

template <bool PREFETCH_IDS>
__global__ __launch_bounds__(kProbeWaves* kWave, 2) void stream_read_kernel(const char* base_a, const char* base_b,
                                                                            const int32_t* page_ids, int64_t pages,
                                                                            int32_t page_bytes, uint32_t* sink) {
  const int lane = threadIdx.x & (kWave - 1);
  const int64_t wave = static_cast<int64_t>(blockIdx.x) * kProbeWaves + (threadIdx.x >> 6);
  const int64_t waves = static_cast<int64_t>(gridDim.x) * kProbeWaves;
  const int pieces = page_bytes / (kWave * 16);  // 1 KB per wave and load instruction
  uint32_t fold = 0;
  const int64_t runs = base_b != nullptr ? 2 * pages : pages;  // the two pools' copies of a page one after the other
  auto page_of = [&](int64_t i) {
    const int64_t index = base_b != nullptr ? i >> 1 : i;
    return page_ids != nullptr ? static_cast<int64_t>(page_ids[index]) : index;
  };
  // PREFETCH_IDS: the id of the wave's next run is requested in front of the current run's loads (as the decode
  // kernel requests block ids a tile ahead), so no run starts with a dependent fetch
  int64_t next_page = (PREFETCH_IDS && wave < runs) ? page_of(wave) : 0;
  for (int64_t i = wave; i < runs; i += waves) {
    int64_t page;
    if constexpr (PREFETCH_IDS) {
      page = next_page;
      next_page = page_of(i + waves < runs ? i + waves : i);
    } else {
      page = page_of(i);
    }
    const char* src = ((base_b != nullptr && (i & 1)) ? base_b : base_a) + page * page_bytes + lane * 16;
    for (int j = 0; j < pieces; j += kProbeLoads) {
      uint4_t v[kProbeLoads];
#pragma unroll
      for (int u = 0; u < kProbeLoads; ++u)
        v[u] = *reinterpret_cast<const uint4_t*>(src + static_cast<int64_t>(min(j + u, pieces - 1)) * kWave * 16);
#pragma unroll
      for (int u = 0; u < kProbeLoads; ++u) fold ^= v[u][0] ^ v[u][1] ^ v[u][2] ^ v[u][3];
    }
  }
  if (fold == 0x9e3779b9u) sink[0] = fold;  // practically never: the store only keeps the loads alive
}

}  // namespace
}  // namespace areno

extern "C" int areno_hip_probe_stream_read(const void* base_a, const void* base_b, const int32_t* page_ids, int64_t pages,
                                           int32_t page_bytes, int32_t prefetch_ids, void* sink, void* stream) {
  const char* op = "areno_hip_probe_stream_read";
  if (base_a == nullptr || sink == nullptr || pages < 0 || page_bytes < 1024 || page_bytes % 1024 != 0)
    return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: NULL pointer, or page_bytes not a positive multiple of 1024", op);
  if (reinterpret_cast<uintptr_t>(base_a) % 16 != 0 || reinterpret_cast<uintptr_t>(base_b) % 16 != 0)
    return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: the pools must be 16-byte aligned", op);
  if (pages == 0) return ARENO_OK;
  const dim3 grid(areno::kProbeWorkgroups), block(areno::kProbeWaves * areno::kWave);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (prefetch_ids != 0 && page_ids != nullptr) {
    hipLaunchKernelGGL(areno::stream_read_kernel<true>, grid, block, 0, s, static_cast<const char*>(base_a),
                       static_cast<const char*>(base_b), page_ids, pages, page_bytes, static_cast<uint32_t*>(sink));
  } else {
    hipLaunchKernelGGL(areno::stream_read_kernel<false>, grid, block, 0, s, static_cast<const char*>(base_a),
                       static_cast<const char*>(base_b), page_ids, pages, page_bytes, static_cast<uint32_t*>(sink));
  }
  return areno::check_launch(op);
}
