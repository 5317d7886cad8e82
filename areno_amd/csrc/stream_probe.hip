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

// Measurement aid: the rate at which the matrix cores take one shape of product when nothing else is asked of them.
// Every wave issues `iters` rounds of independent products on register operands (8 accumulators of 16 x 16, or 4 of
// 32 x 32: the same 32 accumulation registers per lane); 1 024 workgroups of four waves.
typedef __attribute__((ext_vector_type(8))) __bf16 probe_bf16x8;
typedef __attribute__((ext_vector_type(8))) _Float16 probe_f16x8;
typedef __attribute__((ext_vector_type(4))) float probe_f32x4;
typedef __attribute__((ext_vector_type(16))) float probe_f32x16;
constexpr int kRateWorkgroups = 1024;

template <int SHAPE>  // 0: 16 x 16 x 32 bf16, 1: 32 x 32 x 16 bf16, 2: 16 x 16 x 32 f16, 3: 32 x 32 x 16 f16
__global__ __launch_bounds__(kProbeWaves* kWave) void mfma_rate_kernel(int iters, float* sink) {
  probe_bf16x8 a, b;
  probe_f16x8 ah, bh;
  for (int i = 0; i < 8; ++i) {
    a[i] = static_cast<__bf16>(threadIdx.x * 0.001f + i);
    b[i] = static_cast<__bf16>(threadIdx.x * 0.002f - i);
    ah[i] = static_cast<_Float16>(threadIdx.x * 0.001f + i);
    bh[i] = static_cast<_Float16>(threadIdx.x * 0.002f - i);
  }
  probe_f32x4 small[8];
  probe_f32x16 big[4];
  for (int i = 0; i < 8; ++i) small[i] = probe_f32x4{0.0f, 0.0f, 0.0f, 0.0f};
  for (int i = 0; i < 4; ++i) {
    for (int j = 0; j < 16; ++j) big[i][j] = 0.0f;
  }
  for (int it = 0; it < iters; ++it) {
    if constexpr (SHAPE == 0) {
#pragma unroll
      for (int i = 0; i < 8; ++i) small[i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, small[i], 0, 0, 0);
    } else if constexpr (SHAPE == 1) {
#pragma unroll
      for (int i = 0; i < 4; ++i) big[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, big[i], 0, 0, 0);
    } else if constexpr (SHAPE == 2) {
#pragma unroll
      for (int i = 0; i < 8; ++i) small[i] = __builtin_amdgcn_mfma_f32_16x16x32_f16(ah, bh, small[i], 0, 0, 0);
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) big[i] = __builtin_amdgcn_mfma_f32_32x32x16_f16(ah, bh, big[i], 0, 0, 0);
    }
  }
  float fold = 0.0f;
  for (int i = 0; i < 8; ++i) fold += small[i][0] + small[i][3];
  for (int i = 0; i < 4; ++i) fold += big[i][0] + big[i][15];
  if (fold == 12345.678f) sink[0] = fold;  // practically never: the store only keeps the products alive
}

}  // namespace
}  // namespace areno

extern "C" int64_t areno_hip_probe_mfma_rate(int32_t shape, int32_t iters, void* sink, void* stream) {
  const char* op = "areno_hip_probe_mfma_rate";
  if (shape < 0 || shape > 3 || iters < 1 || sink == nullptr) {
    areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: shape 0..3, iters >= 1 and a sink", op);
    return -1;
  }
  const dim3 grid(areno::kRateWorkgroups), block(areno::kProbeWaves * areno::kWave);
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* out = static_cast<float*>(sink);
  switch (shape) {
    case 0: hipLaunchKernelGGL(areno::mfma_rate_kernel<0>, grid, block, 0, s, iters, out); break;
    case 1: hipLaunchKernelGGL(areno::mfma_rate_kernel<1>, grid, block, 0, s, iters, out); break;
    case 2: hipLaunchKernelGGL(areno::mfma_rate_kernel<2>, grid, block, 0, s, iters, out); break;
    default: hipLaunchKernelGGL(areno::mfma_rate_kernel<3>, grid, block, 0, s, iters, out); break;
  }
  if (areno::check_launch(op) != ARENO_OK) return -1;
  // floating-point operations of the launch: 2 x 16 384 multiply-adds per round and wave in either shape
  return static_cast<int64_t>(areno::kRateWorkgroups) * areno::kProbeWaves * iters * (8LL * 16 * 16 * 32 * 2);
}

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
