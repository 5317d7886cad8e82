// Shared device helpers for the gfx950 paged-attention kernels: 16-bit / 8-bit element
// conversions, wave64 cross-lane primitives and the host-side error plumbing of the C ABI.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/areno_hip.h"

// The kernels are written against two code-generation flags that only the build script passes, together with this
// define: -fno-honor-nans (maxima as bare v_max_f32 / v_max3_f32; inputs may hold NaN in slots no query may see, the
// kernels neither produce nor test for NaN) and packed-FP32 VALU forms off.  A build without them would compile and
// give different code for every maximum, so it is refused here.
#if !defined(ARENO_DEVICE_FLAGS_OK)
#error "build areno_amd/csrc through setup.py: it needs -fno-honor-nans and -Xclang -target-feature -Xclang -packed-fp32-ops (HIP_DEVICE_FLAGS)"
#endif

namespace areno {

constexpr int kWave = 64;

typedef __attribute__((ext_vector_type(2))) _Float16 half2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) float float2_t;
typedef __attribute__((ext_vector_type(4))) float float4_t;
typedef __attribute__((ext_vector_type(4))) uint32_t uint4_t;
typedef __attribute__((ext_vector_type(2))) uint32_t uint2_t;

// ---- scalar conversions ------------------------------------------------------------------

__device__ __forceinline__ float bf16_bits_to_float(uint32_t bits16) {
  return __builtin_bit_cast(float, bits16 << 16);
}

__device__ __forceinline__ uint32_t float_to_bf16_bits(float x) {
  __bf16 h = static_cast<__bf16>(x);  // round to nearest even
  return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, h));
}

__device__ __forceinline__ float f16_bits_to_float(uint32_t bits16) {
  return static_cast<float>(__builtin_bit_cast(_Float16, static_cast<uint16_t>(bits16)));
}

__device__ __forceinline__ uint32_t float_to_f16_bits(float x) {
  _Float16 h = static_cast<_Float16>(x);
  return static_cast<uint32_t>(__builtin_bit_cast(uint16_t, h));
}

// OCP e4m3fn byte -> float (hardware conversion; gfx950 implements the OCP encodings).
__device__ __forceinline__ float fp8_byte_to_float(uint32_t byte) {
  return __builtin_amdgcn_cvt_f32_fp8(byte & 0xffu, 0);
}

// float (already clamped to [-448, 448]) -> OCP e4m3fn byte, round to nearest even.
__device__ __forceinline__ uint32_t float_to_fp8_byte(float x) {
  return static_cast<uint32_t>(__builtin_amdgcn_cvt_pk_fp8_f32(x, x, 0, false)) & 0xffu;
}

// Element `idx` of a row stored with the given dtype, as float.
__device__ __forceinline__ float load_as_float(const void* base, int64_t idx, int dtype) {
  switch (dtype) {
    case ARENO_DT_F32: return static_cast<const float*>(base)[idx];
    case ARENO_DT_F16: return f16_bits_to_float(static_cast<const uint16_t*>(base)[idx]);
    case ARENO_DT_BF16: return bf16_bits_to_float(static_cast<const uint16_t*>(base)[idx]);
    case ARENO_DT_I8: return static_cast<float>(static_cast<const int8_t*>(base)[idx]);
    default: return fp8_byte_to_float(static_cast<const uint8_t*>(base)[idx]);
  }
}

__device__ __forceinline__ void store_from_float(void* base, int64_t idx, int dtype, float x) {
  switch (dtype) {
    case ARENO_DT_F32: static_cast<float*>(base)[idx] = x; break;
    case ARENO_DT_F16: static_cast<uint16_t*>(base)[idx] = static_cast<uint16_t>(float_to_f16_bits(x)); break;
    default: static_cast<uint16_t*>(base)[idx] = static_cast<uint16_t>(float_to_bf16_bits(x)); break;
  }
}

__device__ __forceinline__ float load_scale(const void* base, int64_t idx, int scale_dtype) {
  return scale_dtype == ARENO_DT_F16 ? f16_bits_to_float(static_cast<const uint16_t*>(base)[idx])
                                     : static_cast<const float*>(base)[idx];
}

// ---- wave64 cross-lane -------------------------------------------------------------------

__device__ __forceinline__ float wave_xor(float x, int mask) { return __shfl_xor(x, mask, kWave); }

__device__ __forceinline__ float wave_sum(float x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x += wave_xor(x, m);
  return x;
}

__device__ __forceinline__ float wave_max(float x) {
#pragma unroll
  for (int m = 32; m >= 1; m >>= 1) x = fmaxf(x, wave_xor(x, m));
  return x;
}

// Reductions over the four 16-lane rows of a wave (lanes l, l + 16, l + 32, l + 48), result in all four: the MFMA
// C layout keeps one matrix column in those lanes.  v_permlane16_swap / v_permlane32_swap exchange odd and even rows
// (then upper and lower half) of two registers in the vector ALU, without the LDS round trip of ds_bpermute.  Inline
// asm because the compiler's own lowering of the matching builtins merges the two results; the s_nop covers the
// wait states the swap needs after a VALU write of its operands.
__device__ __forceinline__ void swap_rows16(uint32_t& a, uint32_t& b) {
  asm("s_nop 1\n\tv_permlane16_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}
__device__ __forceinline__ void swap_rows32(uint32_t& a, uint32_t& b) {
  asm("s_nop 1\n\tv_permlane32_swap_b32 %0, %1" : "+v"(a), "+v"(b));
}

// Maxima as plain compiler-visible operations, so that the compiler's hazard handling around matrix-core
// instructions covers them (a VALU write into a register that an MFMA issued a few cycles earlier still reads as its
// C operand needs wait states that only the compiler can place; an inline-asm v_max3_f32 that the register allocator
// put there corrupted scores).  The build passes -fno-honor-nans, which is what lets fmaxf become a bare v_max_f32 /
// v_max3_f32 without a canonicalising self-max in front of every operand; no kernel here produces or tests for NaN.
__device__ __forceinline__ float max_f32(float a, float b) { return __builtin_fmaxf(a, b); }
__device__ __forceinline__ float max3_f32(float a, float b, float c) {
  return __builtin_fmaxf(__builtin_fmaxf(a, b), c);
}
// x *= f in the register x lives in: as a plain multiply under a rarely taken branch the compiler copies whole
// accumulator sets around the branch instead.  The compiler places hazard wait states only for its own instructions,
// not for inline asm: a factor that comes straight out of a transcendental op (v_exp_f32) must pass through
// settled() first, or the first multiply issued behind it reads the register before the result has landed.
__device__ __forceinline__ void scale_in_place(float& x, float f) { asm("v_mul_f32 %0, %1, %0" : "+v"(x) : "v"(f)); }
__device__ __forceinline__ float settled(float x) {
  asm("s_nop 1" : "+v"(x));
  return x;
}

__device__ __forceinline__ float rows_max(float x) {
  uint32_t a = __builtin_bit_cast(uint32_t, x), b = a;
  swap_rows16(a, b);
  const float y = max_f32(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
  a = __builtin_bit_cast(uint32_t, y);
  b = a;
  swap_rows32(a, b);
  return max_f32(__builtin_bit_cast(float, a), __builtin_bit_cast(float, b));
}

__device__ __forceinline__ float rows_sum(float x) {
  uint32_t a = __builtin_bit_cast(uint32_t, x), b = a;
  swap_rows16(a, b);
  const float y = __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b);
  a = __builtin_bit_cast(uint32_t, y);
  b = a;
  swap_rows32(a, b);
  return __builtin_bit_cast(float, a) + __builtin_bit_cast(float, b);
}

// Reductions over the whole wave, result in every lane, without the LDS crossbar (ds_bpermute) that __shfl_xor
// compiles to: four data-parallel-primitive steps inside each row of 16 lanes (quad permutes, then the row's half and
// full mirror), then the two row swaps above.  A third of the latency of six ds_bpermute round trips, which is what a
// kernel made of a few dependent steps per wave (the merge launch) consists of.
template <int CTRL>
__device__ __forceinline__ float dpp_lanes(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xf, 0xf, false));
}
constexpr int kDppQuadSwap1 = 0xb1;      // quad_perm [1, 0, 3, 2]
constexpr int kDppQuadSwap2 = 0x4e;      // quad_perm [2, 3, 0, 1]
constexpr int kDppRowHalfMirror = 0x141;  // lane i of a half row <- lane 7 - i
constexpr int kDppRowMirror = 0x140;      // lane i of a row <- lane 15 - i

__device__ __forceinline__ float wave_max_fast(float x) {
  x = max_f32(x, dpp_lanes<kDppQuadSwap1>(x));
  x = max_f32(x, dpp_lanes<kDppQuadSwap2>(x));
  x = max_f32(x, dpp_lanes<kDppRowHalfMirror>(x));
  x = max_f32(x, dpp_lanes<kDppRowMirror>(x));
  return rows_max(x);
}

__device__ __forceinline__ float wave_sum_fast(float x) {
  x += dpp_lanes<kDppQuadSwap1>(x);
  x += dpp_lanes<kDppQuadSwap2>(x);
  x += dpp_lanes<kDppRowHalfMirror>(x);
  x += dpp_lanes<kDppRowMirror>(x);
  return rows_sum(x);
}

__device__ __forceinline__ float fast_exp2(float x) { return __builtin_amdgcn_exp2f(x); }

constexpr float kLog2e = 1.4426950408889634f;

// ---- host side ---------------------------------------------------------------------------

// Division of a token index by the page size as a multiply and a shift: with s = ceil(log2(bs)) and
// magic = floor(2^(30 + s) / bs) + 1, (t * magic) >> (30 + s) == t / bs for every 0 <= t < 2^30 (the error of the
// product is below t / 2^(30 + s) <= 1 / 2^s, which cannot carry a quotient over while (bs - 1) / bs + 1 / 2^s <= 1).
// A kernel takes the high word of the product (__umulhi), so the shift left over is s - 2 and pages of fewer than 4
// tokens are not served this way.
struct PageDivision {
  uint32_t magic;
  int32_t post;
};
inline bool page_division(int64_t block_size, PageDivision* out) {
  if (block_size < 4 || block_size > (1 << 24)) return false;
  int s = 0;
  while ((int64_t{1} << s) < block_size) ++s;
  out->magic = static_cast<uint32_t>((uint64_t{1} << (30 + s)) / static_cast<uint64_t>(block_size) + 1);
  out->post = s - 2;
  return true;
}
void set_error(const char* fmt, ...);
int fail(int status, const char* fmt, ...);
int check_launch(const char* what);
size_t dtype_size(int dtype);
bool is_quantized(int dtype);

}  // namespace areno
