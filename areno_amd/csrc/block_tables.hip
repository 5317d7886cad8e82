// Device-resident page allocator and block tables for the paged KV cache (gfx950).
//
// The reference keeps the free list and the per-sequence page lists as Python lists
// (areno/engine/data/rollout_state.py:55-56), walks them on the host every step and copies a freshly built
// rectangular table to the device (areno/engine/inference.py:561-580).  Here the same state lives in device memory
// and the same transitions run as small integer kernels, so a decode step needs no host walk and no table upload:
//
//   free list        FIFO ring of page ids: pages are taken from the head in request order and given back at the
//                    tail row by row, page by page -- the order of `_free_blocks.pop(0)` / `.extend(blocks)`
//                    (rollout_state.py:151,225, inference.py:656-658), so the ids a row receives are the ones the
//                    reference hands out for the same sequence of requests
//   reserve          "row r must hold n tokens": rollout_state.py:128-151 (prefill chunk admission)
//   ensure_decode    "row r is about to write position p": rollout_state.py:212-225
//   release          inference.py:651-658
//   gather           rectangular [n, max_blocks] table of the given rows, right-padded with the row's last page
//                    (rollout_state.py:282-285, inference.py:573-580) or with the scratch page id = num_blocks
//                    (areno/engine/runtime/decode_graph.py:95,163-174); a negative row gives an all-scratch row
//   prefill_slots    per packed token: position, page id and slot (rollout_state.py:141-149)
//
// Requests of one call are served in index order by ONE workgroup (an exclusive prefix sum over the pages each
// request needs replaces the sequential walk), so the result does not depend on scheduling.  A request that cannot
// be served in full takes what is left, like the reference's loop before it raises, and the call records status
// and the index of the first such request in `state`; later requests of the call get nothing.  Everything is
// 32-bit integer work on a few KB: the kernels are bound by launch latency.

#include "device_common.hpp"

namespace areno {
namespace {

constexpr int kAllocThreads = 1024;

enum { kStateHead = 0, kStateCount = 1, kStateStatus = 2, kStateFirstFail = 3 };

__global__ void block_tables_init_kernel(areno_block_tables bt) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i < bt.num_blocks) bt.free_ring[i] = static_cast<int32_t>(i);
  if (i < bt.max_rows) bt.row_blocks[i] = 0;
  if (i == 0) {
    bt.state[kStateHead] = 0;
    bt.state[kStateCount] = bt.num_blocks;
    bt.state[kStateStatus] = ARENO_BLOCKS_OK;
    bt.state[kStateFirstFail] = -1;
  }
}

// Exclusive prefix sum of one value per thread over the workgroup; returns the offset, *total gets the sum.
__device__ int workgroup_exclusive_scan(int value, int* s_wave, int* total) {
  const int lane = threadIdx.x & (kWave - 1);
  const int wave = threadIdx.x >> 6;
  int incl = value;
#pragma unroll
  for (int off = 1; off < kWave; off <<= 1) {
    const int up = __shfl_up(incl, off, kWave);
    if (lane >= off) incl += up;
  }
  if (lane == kWave - 1) s_wave[wave] = incl;
  __syncthreads();
  int before = 0, sum = 0;
  for (int w = 0; w < kAllocThreads / kWave; ++w) {
    const int v = s_wave[w];
    if (w < wave) before += v;
    sum += v;
  }
  __syncthreads();
  *total = sum;
  return before + incl - value;
}

// True when an earlier request of the call names the same row.  The reference walks the requests one by one and
// would see the row's updated state at the later one; a parallel pass cannot, so the later one is set aside.
// s_rows holds the rows of the current pass of kAllocThreads requests (requests before `base` are read from memory).
// The scan over the earlier entries of the pass has no early exit, so its LDS reads pipeline.
__device__ bool named_earlier(const int64_t* rows, int base, int live, int64_t r, int* s_rows) {
  __syncthreads();  // the previous pass is done with s_rows
  s_rows[threadIdx.x] = static_cast<int>(r);  // rows are < max_rows <= 2^31 - 1, or -1
  __syncthreads();
  const int tid = threadIdx.x;
  const int mine = static_cast<int>(r);
  // uniform over the wave; nothing to scan for waves behind the pass's last request
  const int wave_end = min((tid | (kWave - 1)) + 1, (live + 3) & ~3);
  bool found = false;
#pragma unroll 4
  for (int j = 0; j < wave_end; j += 4) {
    const int4 v = *reinterpret_cast<const int4*>(&s_rows[j]);
    found |= (j + 0 < tid && v.x == mine) | (j + 1 < tid && v.y == mine) | (j + 2 < tid && v.z == mine) |
             (j + 3 < tid && v.w == mine);
  }
  if (r < 0) return false;
  if (found) return true;
  for (int j = 0; j < base; ++j) {
    if (rows[j] == r) return true;
  }
  return false;
}

__device__ void report(const areno_block_tables& bt, int status, int index) {
  atomicMax(&bt.state[kStateStatus], status);
  // first failing request: smallest index; -1 (as unsigned) is the largest value, so a minimum over unsigned works
  atomicMin(reinterpret_cast<unsigned int*>(&bt.state[kStateFirstFail]), static_cast<unsigned int>(index));
}

// Serves the requests of one call in index order; runs in one workgroup of kAllocThreads threads.
// mode 0: amounts[i] = tokens the row must be able to hold; mode 1: amounts[i] = position the row writes next.
__device__ void serve_requests(const areno_block_tables& bt, const int64_t* rows, const int32_t* amounts, int n,
                               int mode, int* s_wave, int* s_rows) {
  const int head = bt.state[kStateHead];
  const int count = bt.state[kStateCount];
  int taken = 0;  // pages asked for by the requests of earlier passes
  for (int base = 0; base < n; base += kAllocThreads) {
    const int i = base + static_cast<int>(threadIdx.x);
    int need = 0, have = 0;
    int64_t r = i < n ? rows[i] : -1;
    if (i < n && (r >= bt.max_rows || (r < 0 && mode == 0))) {
      report(bt, ARENO_BLOCKS_BAD_ROW, i);
      r = -1;
    }
    // (a negative row in a decode request is a padded row of a bucketed batch: nothing to do)
    const bool repeated = named_earlier(rows, base, min(n - base, kAllocThreads), r, s_rows);
    if (r >= 0) {
      const int64_t amount = amounts[i];
      if (repeated) {
        // decode: the earlier request has already opened the page; prefill: one row, two lengths is a caller error
        if (mode == 0) report(bt, ARENO_BLOCKS_BAD_ROW, i);
      } else {
        have = bt.row_blocks[r];
        int64_t required = 0;
        if (mode == 0) {
          required = amount > 0 ? (amount + bt.block_size - 1) / bt.block_size : 0;
        } else if (amount >= 0 && amount % bt.block_size == 0 && have > 0) {
          // only a row that is running and whose next token opens a page asks for one
          required = amount / bt.block_size + 1;
        }
        if (required > bt.max_blocks) {
          report(bt, ARENO_BLOCKS_ROW_FULL, i);
          required = bt.max_blocks;
        }
        need = required > have ? static_cast<int>(required) - have : 0;
      }
    }
    int total;
    const int off = taken + workgroup_exclusive_scan(need, s_wave, &total);
    if (need > 0) {
      const int left = count - off;
      const int grant = left >= need ? need : (left > 0 ? left : 0);
      for (int j = 0; j < grant; ++j)
        bt.table[r * bt.max_blocks + have + j] = bt.free_ring[(head + off + j) % bt.num_blocks];
      bt.row_blocks[r] = have + grant;
      if (grant < need) report(bt, ARENO_BLOCKS_EXHAUSTED, i);
    }
    taken += total;
  }
  __syncthreads();  // every thread has read head / count
  if (threadIdx.x == 0) {
    const int granted = taken < count ? taken : count;
    bt.state[kStateHead] = (head + granted) % bt.num_blocks;
    bt.state[kStateCount] = count - granted;
  }
}

__global__ __launch_bounds__(kAllocThreads) void block_tables_reserve_kernel(areno_block_tables bt, const int64_t* rows,
                                                                            const int32_t* amounts, int n, int mode) {
  __shared__ int s_wave[kAllocThreads / kWave];
  __shared__ __attribute__((aligned(16))) int s_rows[kAllocThreads];
  serve_requests(bt, rows, amounts, n, mode, s_wave, s_rows);
}

__global__ __launch_bounds__(kAllocThreads) void block_tables_release_kernel(areno_block_tables bt, const int64_t* rows,
                                                                            int n) {
  __shared__ int s_wave[kAllocThreads / kWave];
  __shared__ __attribute__((aligned(16))) int s_rows[kAllocThreads];
  const int head = bt.state[kStateHead];
  const int count = bt.state[kStateCount];
  int returned = 0;
  for (int base = 0; base < n; base += kAllocThreads) {
    const int i = base + static_cast<int>(threadIdx.x);
    int have = 0;
    int64_t r = i < n ? rows[i] : -1;
    if (i < n && (r < 0 || r >= bt.max_rows)) {
      report(bt, ARENO_BLOCKS_BAD_ROW, i);
      r = -1;
    }
    // a row named twice gives its pages back once, like dict.pop(row, None)
    const bool repeated = named_earlier(rows, base, min(n - base, kAllocThreads), r, s_rows);
    if (r >= 0 && !repeated) have = bt.row_blocks[r];
    int total;
    const int off = returned + workgroup_exclusive_scan(have, s_wave, &total);
    if (have > 0) {
      const int64_t tail = static_cast<int64_t>(head) + count + off;
      for (int j = 0; j < have; ++j) bt.free_ring[(tail + j) % bt.num_blocks] = bt.table[r * bt.max_blocks + j];
      bt.row_blocks[r] = 0;
    }
    returned += total;
  }
  __syncthreads();
  if (threadIdx.x == 0) bt.state[kStateCount] = count + returned;
}

// Entry (i, c) of the rectangular table of `rows`.  With next_positions (the table of a decode step), a row that
// has no page for the position it writes next -- the pool ran dry when it asked -- becomes a row of scratch ids: the
// decode op then appends its token to the scratch page instead of overwriting slot 0 of the row's last page.
__device__ void gather_entry(const areno_block_tables& bt, const int64_t* rows, const int32_t* next_positions, int i,
                             int c, int pad_mode, int32_t* out) {
  const int64_t r = rows[i];
  int32_t id = bt.num_blocks;  // the scratch page
  if (r >= 0 && r < bt.max_rows) {
    const int have = bt.row_blocks[r];
    const bool unserved = next_positions != nullptr && have > 0 &&
                          static_cast<int64_t>(next_positions[i]) >= static_cast<int64_t>(have) * bt.block_size;
    if (unserved) {
      // parked; the status word already says why (exhausted pool or full row)
    } else if (c < have) {
      id = bt.table[r * bt.max_blocks + c];
    } else if (have > 0 && pad_mode == ARENO_PAD_LAST_BLOCK) {
      id = bt.table[r * bt.max_blocks + have - 1];
    } else if (have == 0 && c == 0) {
      report(bt, ARENO_BLOCKS_BAD_ROW, i);  // the reference refuses an empty row (rollout_state.py:283-284)
    }
  } else if (r >= bt.max_rows && c == 0) {
    report(bt, ARENO_BLOCKS_BAD_ROW, i);
  }
  out[static_cast<int64_t>(i) * bt.max_blocks + c] = id;
}

__global__ void block_tables_gather_kernel(areno_block_tables bt, const int64_t* rows, const int32_t* next_positions,
                                           int n, int pad_mode, int32_t* out) {
  const int c = blockIdx.x * blockDim.x + threadIdx.x;
  if (c < bt.max_blocks) gather_entry(bt, rows, next_positions, blockIdx.y, c, pad_mode, out);
}

__global__ void block_tables_prefill_slots_kernel(areno_block_tables bt, const int64_t* rows, const int32_t* cursors,
                                                  const int32_t* cu_seqlens, int n, int64_t tokens, int64_t* out_ids,
                                                  int64_t* out_offsets, int64_t* out_positions) {
  const int64_t t = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (t >= tokens) return;
  // sequence of packed token t: the largest i with cu_seqlens[i] <= t
  int lo = 0, hi = n;
  while (lo + 1 < hi) {
    const int mid = (lo + hi) >> 1;
    if (cu_seqlens[mid] <= t) {
      lo = mid;
    } else {
      hi = mid;
    }
  }
  const int64_t r = rows[lo];
  const int64_t pos = static_cast<int64_t>(cursors[lo]) + (t - cu_seqlens[lo]);
  const int64_t col = pos / bt.block_size;
  int64_t id = bt.num_blocks;
  if (r >= 0 && r < bt.max_rows && col < bt.row_blocks[r]) {
    id = bt.table[r * bt.max_blocks + col];
  } else {
    report(bt, ARENO_BLOCKS_BAD_ROW, lo);
  }
  out_ids[t] = id;
  out_offsets[t] = pos - col * bt.block_size;
  if (out_positions != nullptr) out_positions[t] = pos;
}

int validate_tables(const areno_block_tables* bt, const char* op) {
  if (bt == nullptr) return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: table descriptor is NULL", op);
  if (bt->table == nullptr || bt->row_blocks == nullptr || bt->free_ring == nullptr || bt->state == nullptr)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: table pointer is NULL", op);
  if (bt->max_rows <= 0 || bt->max_blocks <= 0 || bt->num_blocks <= 0 || bt->block_size <= 0)
    return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: table shape must be positive", op);
  return ARENO_OK;
}

int launch_reserve(const areno_block_tables* bt, const int64_t* rows, const int32_t* amounts, int32_t n, int mode,
                   void* stream, const char* op) {
  if (int rc = validate_tables(bt, op)) return rc;
  if (n < 0) return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: negative request count", op);
  if (n == 0) return ARENO_OK;
  if (rows == nullptr || amounts == nullptr) return fail(ARENO_ERR_INVALID_ARGUMENT, "%s: request pointer is NULL", op);
  hipLaunchKernelGGL(block_tables_reserve_kernel, dim3(1), dim3(kAllocThreads), 0, static_cast<hipStream_t>(stream),
                     *bt, rows, amounts, n, mode);
  return check_launch(op);
}


int launch_gather(const areno_block_tables* bt, const int64_t* rows, const int32_t* next_positions, int32_t n,
                  int32_t pad_mode, int32_t* out_table, void* stream, const char* op) {
  if (int rc = areno::validate_tables(bt, op)) return rc;
  if (n < 0 || n > 65535) return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: row count %d out of range", op, n);
  if (pad_mode != ARENO_PAD_LAST_BLOCK && pad_mode != ARENO_PAD_SCRATCH_BLOCK)
    return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: unknown pad mode %d", op, pad_mode);
  if (n == 0) return ARENO_OK;
  if (rows == nullptr || out_table == nullptr)
    return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: rows / out_table is NULL", op);
  const unsigned col_blocks = static_cast<unsigned>((bt->max_blocks + 255) / 256);
  hipLaunchKernelGGL(areno::block_tables_gather_kernel, dim3(col_blocks, static_cast<unsigned>(n)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), *bt, rows, next_positions, n, pad_mode, out_table);
  return areno::check_launch(op);
}
}  // namespace
}  // namespace areno

extern "C" int areno_hip_block_tables_init(const areno_block_tables* bt, void* stream) {
  const char* op = "areno_hip_block_tables_init";
  if (int rc = areno::validate_tables(bt, op)) return rc;
  const int64_t items = bt->num_blocks > bt->max_rows ? bt->num_blocks : bt->max_rows;
  hipLaunchKernelGGL(areno::block_tables_init_kernel, dim3(static_cast<unsigned>((items + 255) / 256)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), *bt);
  return areno::check_launch(op);
}

extern "C" int areno_hip_block_tables_reserve(const areno_block_tables* bt, const int64_t* rows,
                                              const int32_t* token_counts, int32_t n, void* stream) {
  return areno::launch_reserve(bt, rows, token_counts, n, 0, stream, "areno_hip_block_tables_reserve");
}

extern "C" int areno_hip_block_tables_ensure_decode(const areno_block_tables* bt, const int64_t* rows,
                                                    const int32_t* next_positions, int32_t n, void* stream) {
  return areno::launch_reserve(bt, rows, next_positions, n, 1, stream, "areno_hip_block_tables_ensure_decode");
}

extern "C" int areno_hip_block_tables_release(const areno_block_tables* bt, const int64_t* rows, int32_t n,
                                              void* stream) {
  const char* op = "areno_hip_block_tables_release";
  if (int rc = areno::validate_tables(bt, op)) return rc;
  if (n < 0) return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: negative row count", op);
  if (n == 0) return ARENO_OK;
  if (rows == nullptr) return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: rows is NULL", op);
  hipLaunchKernelGGL(areno::block_tables_release_kernel, dim3(1), dim3(areno::kAllocThreads), 0,
                     static_cast<hipStream_t>(stream), *bt, rows, n);
  return areno::check_launch(op);
}

extern "C" int areno_hip_block_tables_gather(const areno_block_tables* bt, const int64_t* rows, int32_t n,
                                             int32_t pad_mode, int32_t* out_table, void* stream) {
  return areno::launch_gather(bt, rows, nullptr, n, pad_mode, out_table, stream, "areno_hip_block_tables_gather");
}


extern "C" int areno_hip_block_tables_decode_step(const areno_block_tables* bt, const int64_t* rows,
                                                  const int32_t* next_positions, int32_t n, int32_t pad_mode,
                                                  int32_t* out_table, void* stream) {
  const char* op = "areno_hip_block_tables_decode_step";
  if (int rc = areno::validate_tables(bt, op)) return rc;
  if (n < 0) return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: negative row count", op);
  if (pad_mode != ARENO_PAD_LAST_BLOCK && pad_mode != ARENO_PAD_SCRATCH_BLOCK)
    return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: unknown pad mode %d", op, pad_mode);
  if (n == 0) return ARENO_OK;
  if (rows == nullptr || next_positions == nullptr || out_table == nullptr)
    return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: argument pointer is NULL", op);
  // (one workgroup doing both was measured slower than the two launches: its table pass is a chain of dependent
  // loads that the many workgroups of the gather kernel overlap)
  if (int rc = areno_hip_block_tables_ensure_decode(bt, rows, next_positions, n, stream)) return rc;
  // rows the pool could not serve come out as rows of scratch ids (see gather_entry)
  return areno::launch_gather(bt, rows, next_positions, n, pad_mode, out_table, stream, op);
}

extern "C" int areno_hip_block_tables_prefill_slots(const areno_block_tables* bt, const int64_t* rows,
                                                    const int32_t* cursors, const int32_t* cu_seqlens, int32_t n,
                                                    int64_t tokens, int64_t* out_block_ids, int64_t* out_block_offsets,
                                                    int64_t* out_positions, void* stream) {
  const char* op = "areno_hip_block_tables_prefill_slots";
  if (int rc = areno::validate_tables(bt, op)) return rc;
  if (n < 0 || tokens < 0) return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: negative count", op);
  if (n == 0 || tokens == 0) return ARENO_OK;
  if (rows == nullptr || cursors == nullptr || cu_seqlens == nullptr || out_block_ids == nullptr ||
      out_block_offsets == nullptr)
    return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: argument pointer is NULL", op);
  const int64_t blocks = (tokens + 255) / 256;
  if (blocks > 0x7fffffffLL) return areno::fail(ARENO_ERR_INVALID_ARGUMENT, "%s: too many tokens", op);
  hipLaunchKernelGGL(areno::block_tables_prefill_slots_kernel, dim3(static_cast<unsigned>(blocks)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), *bt, rows, cursors, cu_seqlens, n, tokens, out_block_ids,
                     out_block_offsets, out_positions);
  return areno::check_launch(op);
}
