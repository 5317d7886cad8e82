// Per-row KV quantizer shared by the cache writers: one wave64 holds a (token, kv head) row as floats, element
// idx = lane + 64 e in x[e]; the row's abs-max gives its scale, codes and scale go to the paged address.
//
// Closed forms (bit-exact contract; IEEE fp32 division, round half to even):
//   int8: s = fp16(min(absmax / 127, 65504)); s == 0 -> 1; code = clamp(rint(x / float(s)), -127, 127)
//   fp8 : s = absmax / 448 (fp32);            s == 0 -> 1; code = e4m3fn(clamp(x / s, -448, 448))
#pragma once

#include "device_common.hpp"

namespace areno {

constexpr int kMaxPerLane = 8;  // head_dim <= 512

__host__ __device__ inline bool is_quantized_dtype(int dtype) {
  return dtype == ARENO_DT_I8 || dtype == ARENO_DT_FP8_E4M3;
}

// One row of EPW elements per lane (element idx = lane + 64 e, zeros behind the head's end): codes and scale by the
// closed forms above, stored at cache row dst_row when `store` is set; xhat[e] receives what a reader of the page
// sees for the element (code times the scale as stored).
template <int EPW>
__device__ __forceinline__ void quantize_row(const float (&x)[EPW], int lane, int d, int64_t dst_row, void* cache,
                                             void* scale, int cache_dtype, int scale_dtype, bool store,
                                             float (&xhat)[EPW]) {
  const int64_t dst_base = dst_row * d;
  float amax = 0.0f;
#pragma unroll
  for (int e = 0; e < EPW; ++e) amax = fmaxf(amax, fabsf(x[e]));
  amax = wave_max_fast(amax);
  if (cache_dtype == ARENO_DT_I8) {
    const _Float16 s16 = static_cast<_Float16>(fminf(amax / 127.0f, 65504.0f));
    const _Float16 s16_fixed = (s16 == static_cast<_Float16>(0.0f)) ? static_cast<_Float16>(1.0f) : s16;
    const float s = static_cast<float>(s16_fixed);
    int8_t* out = static_cast<int8_t*>(cache);
#pragma unroll
    for (int e = 0; e < EPW; ++e) {
      const int idx = lane + e * kWave;
      const float code = fminf(fmaxf(rintf(x[e] / s), -127.0f), 127.0f);
      xhat[e] = code * s;
      if (store && idx < d) out[dst_base + idx] = static_cast<int8_t>(static_cast<int>(code));
    }
    if (store && lane == 0) {
      if (scale_dtype == ARENO_DT_F16) {
        static_cast<uint16_t*>(scale)[dst_row] = __builtin_bit_cast(uint16_t, s16_fixed);
      } else {
        static_cast<float*>(scale)[dst_row] = s;
      }
    }
  } else {
    float s = amax / 448.0f;
    if (s == 0.0f) s = 1.0f;
    const float s_stored = scale_dtype == ARENO_DT_F16 ? f16_bits_to_float(float_to_f16_bits(s)) : s;
    uint8_t* out = static_cast<uint8_t*>(cache);
#pragma unroll
    for (int e = 0; e < EPW; ++e) {
      const int idx = lane + e * kWave;
      const float y = fminf(fmaxf(x[e] / s, -448.0f), 448.0f);
      const uint32_t byte = float_to_fp8_byte(y);
      xhat[e] = fp8_byte_to_float(byte) * s_stored;
      if (store && idx < d) out[dst_base + idx] = static_cast<uint8_t>(byte);
    }
    if (store && lane == 0) {
      if (scale_dtype == ARENO_DT_F16) {
        static_cast<uint16_t*>(scale)[dst_row] = static_cast<uint16_t>(float_to_f16_bits(s));
      } else {
        static_cast<float*>(scale)[dst_row] = s;
      }
    }
  }
}

__device__ __forceinline__ void quantize_store_row(const float (&x)[kMaxPerLane], int lane, int d, int64_t dst_row,
                                                   void* cache, void* scale, int cache_dtype, int scale_dtype) {
  float unused[kMaxPerLane];
  quantize_row<kMaxPerLane>(x, lane, d, dst_row, cache, scale, cache_dtype, scale_dtype, true, unused);
}

// The same closed forms for a row held by a group of LPR adjacent lanes, 8 consecutive elements per lane (lane `sub`
// of the group holds elements 8 sub .. 8 sub + 7; head_dim = 8 LPR): 16-byte accesses instead of one element per
// lane.  `amax` is the row's abs-max, already combined over the group.  16-bit caches get the values rounded to the
// cache dtype.
__device__ __forceinline__ uint32_t pack_two_16(float lo, float hi, int dtype) {
  return dtype == ARENO_DT_BF16 ? (float_to_bf16_bits(lo) | (float_to_bf16_bits(hi) << 16))
                                : (float_to_f16_bits(lo) | (float_to_f16_bits(hi) << 16));
}

template <int LPR>
__device__ __forceinline__ float lane_group_max(float x) {
#pragma unroll
  for (int m = 1; m < LPR; m <<= 1) x = fmaxf(x, wave_xor(x, m));
  return x;
}

// x[j] / s for the eight elements a lane holds and the row's one divisor, rounded as the IEEE division rounds: the
// steps of the correctly rounded sequence (reciprocal, one Newton step on it, quotient, two residual corrections;
// what the compiler emits per division, less the rescaling of extreme operands) with the reciprocal's part done
// once for the row: 5 instructions per element instead of 12.  Divisors outside 2^-60 .. 2^60, infinities and NaN, and
// rows with an infinite element (`amax` is the row's abs-max) take the plain division.  Quotients below 2^-20 in magnitude may differ from the plain division's in their last
// bits; every code below rounds them to a zero of the right sign.
__device__ __forceinline__ void divide_row_slice(const float (&x)[8], float s, float amax, float (&q)[8]) {
  // (an infinite element would come out of the corrections as NaN: a row that holds one takes the plain division)
  if (s >= 0x1p-60f && s <= 0x1p60f && amax <= 0x1.fffffep127f) {
    const float r0 = __builtin_amdgcn_rcpf(s);
    const float r = fmaf(fmaf(-s, r0, 1.0f), r0, r0);
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      float t = x[j] * r;
      t = fmaf(fmaf(-s, t, x[j]), r, t);
      t = fmaf(fmaf(-s, t, x[j]), r, t);
      q[j] = copysignf(t, x[j]);  // -0 / s is -0; the corrections above would leave +0
    }
  } else {
#pragma unroll
    for (int j = 0; j < 8; ++j) q[j] = x[j] / s;
  }
}

__device__ __forceinline__ void store_row_slice(const float (&x)[8], float amax, int sub, int64_t dst_row, int d,
                                                void* cache, void* scale, int cache_dtype, int scale_dtype) {
  const int64_t dst_elem = dst_row * d + sub * 8;
  if (cache_dtype == ARENO_DT_I8) {
    const _Float16 s16 = static_cast<_Float16>(fminf(amax / 127.0f, 65504.0f));
    const _Float16 s16_fixed = (s16 == static_cast<_Float16>(0.0f)) ? static_cast<_Float16>(1.0f) : s16;
    const float s = static_cast<float>(s16_fixed);
    float q[8];
    divide_row_slice(x, s, amax, q);
    uint32_t words[2] = {0u, 0u};
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      const float code = fminf(fmaxf(rintf(q[j]), -127.0f), 127.0f);
      words[j / 4] |= (static_cast<uint32_t>(static_cast<int>(code)) & 0xffu) << (8 * (j & 3));
    }
    *reinterpret_cast<uint2_t*>(static_cast<char*>(cache) + dst_elem) = uint2_t{words[0], words[1]};
    if (sub == 0) {
      if (scale_dtype == ARENO_DT_F16) {
        static_cast<uint16_t*>(scale)[dst_row] = __builtin_bit_cast(uint16_t, s16_fixed);
      } else {
        static_cast<float*>(scale)[dst_row] = s;
      }
    }
  } else if (cache_dtype == ARENO_DT_FP8_E4M3) {
    float s = amax / 448.0f;
    if (s == 0.0f) s = 1.0f;
    float q[8];
    divide_row_slice(x, s, amax, q);
#pragma unroll
    for (int j = 0; j < 8; ++j) q[j] = fminf(fmaxf(q[j], -448.0f), 448.0f);
    // two codes per conversion, into the low or the high half of the word
    int w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], 0, false);
    w0 = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], w0, true);
    int w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[4], q[5], 0, false);
    w1 = __builtin_amdgcn_cvt_pk_fp8_f32(q[6], q[7], w1, true);
    *reinterpret_cast<uint2_t*>(static_cast<char*>(cache) + dst_elem) =
        uint2_t{static_cast<uint32_t>(w0), static_cast<uint32_t>(w1)};
    if (sub == 0) {
      if (scale_dtype == ARENO_DT_F16) {
        static_cast<uint16_t*>(scale)[dst_row] = static_cast<uint16_t>(float_to_f16_bits(s));
      } else {
        static_cast<float*>(scale)[dst_row] = s;
      }
    }
  } else {
    const uint4_t packed = {pack_two_16(x[0], x[1], cache_dtype), pack_two_16(x[2], x[3], cache_dtype),
                            pack_two_16(x[4], x[5], cache_dtype), pack_two_16(x[6], x[7], cache_dtype)};
    *reinterpret_cast<uint4_t*>(static_cast<char*>(cache) + dst_elem * 2) = packed;
  }
}

}  // namespace areno
