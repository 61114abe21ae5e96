// Row-wise e4m3 quantiser (one power-of-two scale per 128-element row).
// HBM-bound: reads 2 B and writes 1 B per element plus 4 B per row; one 64-lane wave per row
// group, each lane handling 8 consecutive elements (16-byte loads, 8-byte stores).
#include "dsa_common.h"

namespace {

__device__ __forceinline__ float wave_max16(float v) {   // max over the 16 lanes sharing a row
  v = fmaxf(v, __shfl_xor(v, 1, 64));
  v = fmaxf(v, __shfl_xor(v, 2, 64));
  v = fmaxf(v, __shfl_xor(v, 4, 64));
  v = fmaxf(v, __shfl_xor(v, 8, 64));
  return v;
}

// cols == 128: 16 lanes per row, 4 rows per wave, 16 rows per 256-thread block.
__global__ __launch_bounds__(256) void quant128_kernel(const uint4* __restrict__ x, uint2* __restrict__ x8,
                                                       float* __restrict__ scale_inv, int64_t rows,
                                                       float eps, int pow2, const float* __restrict__ w_in,
                                                       float w_factor, float* __restrict__ w_scaled) {
  int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  int sub = threadIdx.x & 15;
  bool live = row < rows;
  uint4 raw = live ? x[row * 16 + sub] : make_uint4(0, 0, 0, 0);
  unsigned w[4] = {raw.x, raw.y, raw.z, raw.w};
  float v[8];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    v[2 * i] = __builtin_bit_cast(float, w[i] << 16);
    v[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
  }
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) amax = fmaxf(amax, fabsf(v[i]));
  amax = wave_max16(amax);
  amax = fmaxf(amax, eps);
  float scale = 448.0f / amax;                       // correctly rounded fp32 division
  if (pow2) scale = __builtin_bit_cast(float, __builtin_bit_cast(unsigned, scale) & 0xff800000u);
  float q[8];
#pragma unroll
  for (int i = 0; i < 8; i++) q[i] = fminf(fmaxf(v[i] * scale, -448.0f), 448.0f);  // cvt does not saturate
  int lo = 0, hi = 0;
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], lo, false);
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], lo, true);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(q[4], q[5], hi, false);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(q[6], q[7], hi, true);
  if (live) {
    x8[row * 16 + sub] = make_uint2((unsigned)lo, (unsigned)hi);
    if (sub == 0) {
      const float si = 1.0f / scale;
      scale_inv[row] = si;
      if (w_scaled) w_scaled[row] = (w_in[row] * si) * w_factor;      // two roundings, as two separate multiplications
    }
  }
}

// Hadamard rotation of a 128-element row (Sylvester order, scaled by 128^-0.5, rounded to bf16 as the
// unfused sequence "fp32 product with the Hadamard matrix -> bf16" does) followed by the same
// quantiser.  The butterfly runs over the 7 index bits: 3 inside a lane's 8 elements, 4 across the
// 16 lanes of a row.  Either output may be absent (x8 == nullptr: rotation only; y == nullptr:
// quantised payload only).
__global__ __launch_bounds__(256) void rotate_quant128_kernel(const uint4* __restrict__ x, uint2* __restrict__ x8,
                                                              float* __restrict__ scale_inv, uint4* __restrict__ y,
                                                              int64_t rows, float eps, int pow2,
                                                              const float* __restrict__ w_in, float w_factor,
                                                              float* __restrict__ w_scaled) {
  int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  int sub = threadIdx.x & 15;
  bool live = row < rows;
  uint4 raw = live ? x[row * 16 + sub] : make_uint4(0, 0, 0, 0);
  unsigned w[4] = {raw.x, raw.y, raw.z, raw.w};
  float v[8];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    v[2 * i] = __builtin_bit_cast(float, w[i] << 16);
    v[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
  }
#pragma unroll
  for (int m = 1; m < 8; m <<= 1)
#pragma unroll
    for (int i = 0; i < 8; i++)
      if (!(i & m)) { const float a = v[i], b = v[i | m]; v[i] = a + b; v[i | m] = a - b; }
#pragma unroll
  for (int m = 1; m < 16; m <<= 1)
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const float o = __shfl_xor(v[i], m, 64);
      v[i] = (sub & m) ? o - v[i] : v[i] + o;
    }
  unsigned yb[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const unsigned lo = f32_to_bf16_bits(v[2 * i] * 0.08838834764831845f), hi = f32_to_bf16_bits(v[2 * i + 1] * 0.08838834764831845f);
    yb[i] = lo | (hi << 16);
    v[2 * i] = __builtin_bit_cast(float, lo << 16);
    v[2 * i + 1] = __builtin_bit_cast(float, hi << 16);
  }
  if (live && y) y[row * 16 + sub] = make_uint4(yb[0], yb[1], yb[2], yb[3]);
  if (!x8) return;
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) amax = fmaxf(amax, fabsf(v[i]));
  amax = wave_max16(amax);
  amax = fmaxf(amax, eps);
  float scale = 448.0f / amax;
  if (pow2) scale = __builtin_bit_cast(float, __builtin_bit_cast(unsigned, scale) & 0xff800000u);
  float q[8];
#pragma unroll
  for (int i = 0; i < 8; i++) q[i] = fminf(fmaxf(v[i] * scale, -448.0f), 448.0f);
  int lo = 0, hi = 0;
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], lo, false);
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], lo, true);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(q[4], q[5], hi, false);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(q[6], q[7], hi, true);
  if (live) {
    x8[row * 16 + sub] = make_uint2((unsigned)lo, (unsigned)hi);
    if (sub == 0) {
      const float si = 1.0f / scale;
      scale_inv[row] = si;
      if (w_scaled) w_scaled[row] = (w_in[row] * si) * w_factor;      // two roundings, as two separate multiplications
    }
  }
}


// The indexer front end behind its projections, one pass over a 128-element row:
//   LN    (key rows)  y = ((x - mean) * rstd) * gamma + beta, statistics in fp32, rounded to bf16
//   ROPE              rotation of the leading 64 elements by the row's position (pairs adjacent or split,
//                     the formula and rounding of rope_rows_kernel in rope.hip), rounded to bf16
//   rotation          Hadamard butterfly * 128^-0.5, rounded to bf16 (as rotate_quant128_kernel)
//   quantiser         power-of-two scale, e4m3 payload, optionally weights * scale_inv * factor
// Every stage rounds where the separate operations round, so the payload is that of the unfused sequence.
// Sums run in a fixed order (a lane's 8 elements in sequence, then the 16 lanes of a row by xor 1, 2, 4, 8).
template <bool LN, int PAIRING>   // PAIRING: -1 no rotary part, 0 adjacent pairs, 1 split pairs (i, i + 32)
__global__ __launch_bounds__(256) void indexer_front128_kernel(
    const uint4* __restrict__ x, int64_t rows, int rows_per_token, const float* __restrict__ ln_w,
    const float* __restrict__ ln_b, float ln_eps, const void* __restrict__ cos_t, const void* __restrict__ sin_t,
    int cs_f32, const int* __restrict__ positions, int batch, int rotate, uint2* __restrict__ x8,
    float* __restrict__ scale_inv, uint4* __restrict__ y, float eps, int pow2, const float* __restrict__ w_in,
    float w_factor, float* __restrict__ w_scaled) {
#pragma clang fp contract(off)
  const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  const int sub = threadIdx.x & 15;
  const bool live = row < rows;
  const uint4 raw = live ? x[row * 16 + sub] : make_uint4(0, 0, 0, 0);
  const unsigned w[4] = {raw.x, raw.y, raw.z, raw.w};
  float v[8];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    v[2 * i] = __builtin_bit_cast(float, w[i] << 16);
    v[2 * i + 1] = __builtin_bit_cast(float, w[i] & 0xffff0000u);
  }
  auto row_sum = [&](const float (&t)[8]) {
    float s = t[0];
#pragma unroll
    for (int i = 1; i < 8; i++) s = s + t[i];
#pragma unroll
    for (int m = 1; m < 16; m <<= 1) s = s + __shfl_xor(s, m, 64);
    return s;
  };
  auto round_bf16 = [&]() {
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = bf16_bits_to_f32(f32_to_bf16_bits(v[i]));
  };
  if (LN) {
    const float mean = row_sum(v) * 0.0078125f;
    float d[8], d2[8];
#pragma unroll
    for (int i = 0; i < 8; i++) { d[i] = v[i] - mean; d2[i] = d[i] * d[i]; }
    const float var = row_sum(d2) * 0.0078125f;
    const float rstd = 1.0f / sqrtf(var + ln_eps);
    const f32x4 g0 = *(const f32x4*)(ln_w + 8 * sub), g1 = *(const f32x4*)(ln_w + 8 * sub + 4);
    const f32x4 b0 = *(const f32x4*)(ln_b + 8 * sub), b1 = *(const f32x4*)(ln_b + 8 * sub + 4);
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = (d[i] * rstd) * (i < 4 ? g0[i] : g1[i - 4]) + (i < 4 ? b0[i] : b1[i - 4]);
    round_bf16();
  }
  if (PAIRING >= 0) {
    const int64_t tok = row / rows_per_token;
    const int64_t pos = live ? (positions ? positions[tok] : tok / batch) : 0;
    auto table8 = [&](const void* t, int col, float (&o)[8]) {     // 8 consecutive entries of the position's row
      if (cs_f32) {
        const f32x4 a = *(const f32x4*)((const float*)t + pos * 64 + col), b = *(const f32x4*)((const float*)t + pos * 64 + col + 4);
#pragma unroll
        for (int i = 0; i < 4; i++) { o[i] = a[i]; o[4 + i] = b[i]; }
      } else {
        const uint4 a = *(const uint4*)((const unsigned short*)t + pos * 64 + col);
        const unsigned u[4] = {a.x, a.y, a.z, a.w};
#pragma unroll
        for (int i = 0; i < 4; i++) { o[2 * i] = __builtin_bit_cast(float, u[i] << 16); o[2 * i + 1] = __builtin_bit_cast(float, u[i] & 0xffff0000u); }
      }
    };
    if (PAIRING == 0) {
      if (sub < 8) {            // pairs (2i, 2i + 1) inside the lane; cos / sin indexed like the elements
        float c[8], s[8];
        table8(cos_t, 8 * sub, c);
        table8(sin_t, 8 * sub, s);
#pragma unroll
        for (int i = 0; i < 8; i += 2) {
          const float x1 = v[i], x2 = v[i + 1];
          v[i] = x1 * c[i] - x2 * s[i];
          v[i + 1] = x2 * c[i + 1] + x1 * s[i + 1];
        }
      }
    } else {
      float o[8];               // element e of lane s pairs with element e of lane s ^ 4 (lanes 0..7 hold the 64 rotary elements)
#pragma unroll
      for (int i = 0; i < 8; i++) o[i] = __shfl_xor(v[i], 4, 64);
      if (sub < 8) {
        float c[8], s[8];
        table8(cos_t, 8 * sub, c);
        table8(sin_t, 8 * sub, s);
#pragma unroll
        for (int i = 0; i < 8; i++) v[i] = sub < 4 ? v[i] * c[i] - o[i] * s[i] : v[i] * c[i] + o[i] * s[i];
      }
    }
    round_bf16();
  }
  unsigned yb[4];
  if (rotate) {
#pragma unroll
    for (int m = 1; m < 8; m <<= 1)
#pragma unroll
      for (int i = 0; i < 8; i++)
        if (!(i & m)) { const float a = v[i], b = v[i | m]; v[i] = a + b; v[i | m] = a - b; }
#pragma unroll
    for (int m = 1; m < 16; m <<= 1)
#pragma unroll
      for (int i = 0; i < 8; i++) {
        const float o = __shfl_xor(v[i], m, 64);
        v[i] = (sub & m) ? o - v[i] : v[i] + o;
      }
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = v[i] * 0.08838834764831845f;
    round_bf16();
  }
#pragma unroll
  for (int i = 0; i < 4; i++) yb[i] = (__builtin_bit_cast(unsigned, v[2 * i]) >> 16) | (__builtin_bit_cast(unsigned, v[2 * i + 1]) & 0xffff0000u);
  if (live && y) y[row * 16 + sub] = make_uint4(yb[0], yb[1], yb[2], yb[3]);
  if (!x8) return;
  float amax = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) amax = fmaxf(amax, fabsf(v[i]));
  amax = wave_max16(amax);
  amax = fmaxf(amax, eps);
  float scale = 448.0f / amax;
  if (pow2) scale = __builtin_bit_cast(float, __builtin_bit_cast(unsigned, scale) & 0xff800000u);
  float q[8];
#pragma unroll
  for (int i = 0; i < 8; i++) q[i] = fminf(fmaxf(v[i] * scale, -448.0f), 448.0f);
  int lo = 0, hi = 0;
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(q[0], q[1], lo, false);
  lo = __builtin_amdgcn_cvt_pk_fp8_f32(q[2], q[3], lo, true);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(q[4], q[5], hi, false);
  hi = __builtin_amdgcn_cvt_pk_fp8_f32(q[6], q[7], hi, true);
  if (live) {
    x8[row * 16 + sub] = make_uint2((unsigned)lo, (unsigned)hi);
    if (sub == 0) {
      const float si = 1.0f / scale;
      scale_inv[row] = si;
      if (w_scaled) w_scaled[row] = (w_in[row] * si) * w_factor;
    }
  }
}

}  // namespace

extern "C" int dsa_rotate_quant_e4m3(const void* x, int64_t rows, int cols, void* x8, float* scale_inv, void* y,
                                     float eps, int pow2, void* stream) {
  DSA_REQUIRE(cols == 128, "dsa_rotate_quant_e4m3: only rows of 128 elements are supported, got %d", cols);
  DSA_REQUIRE(rows >= 0, "dsa_rotate_quant_e4m3: negative row count");
  DSA_REQUIRE(x8 != nullptr || y != nullptr, "dsa_rotate_quant_e4m3: no output requested");
  DSA_REQUIRE(x8 == nullptr || scale_inv != nullptr, "dsa_rotate_quant_e4m3: payload without scales");
  DSA_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)x8 % 8) == 0 && ((uintptr_t)y % 16) == 0,
              "dsa_rotate_quant_e4m3: misaligned pointer");
  if (rows == 0) return DSA_OK;
  int64_t blocks = (rows + 15) / 16;
  DSA_REQUIRE(blocks < (1ll << 31), "dsa_rotate_quant_e4m3: too many rows");
  rotate_quant128_kernel<<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(
      (const uint4*)x, (uint2*)x8, scale_inv, (uint4*)y, rows, eps, pow2, nullptr, 0.f, nullptr);
  DSA_CHECK_LAUNCH("dsa_rotate_quant_e4m3");
  return DSA_OK;
}

extern "C" int dsa_quant_rowwise_e4m3(const void* x, int64_t rows, int cols, void* x8, float* scale_inv,
                                      float eps, int pow2, void* stream) {
  DSA_REQUIRE(cols == 128, "dsa_quant_rowwise_e4m3: only rows of 128 elements are supported, got %d", cols);
  DSA_REQUIRE(rows >= 0, "dsa_quant_rowwise_e4m3: negative row count");
  DSA_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)x8 % 8) == 0, "dsa_quant_rowwise_e4m3: misaligned pointer");
  if (rows == 0) return DSA_OK;
  int64_t blocks = (rows + 15) / 16;
  DSA_REQUIRE(blocks < (1ll << 31), "dsa_quant_rowwise_e4m3: too many rows");
  quant128_kernel<<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(
      (const uint4*)x, (uint2*)x8, scale_inv, rows, eps, pow2, nullptr, 0.f, nullptr);
  DSA_CHECK_LAUNCH("dsa_quant_rowwise_e4m3");
  return DSA_OK;
}

extern "C" int dsa_quant_rowwise_e4m3_weights(const void* x, int64_t rows, int cols, void* x8, float* scale_inv,
                                              float eps, int pow2, int rotate, const float* weights, float factor,
                                              float* weight_scaled, void* stream) {
  DSA_REQUIRE(cols == 128, "dsa_quant_rowwise_e4m3_weights: only rows of 128 elements are supported, got %d", cols);
  DSA_REQUIRE(rows >= 0, "dsa_quant_rowwise_e4m3_weights: negative row count");
  DSA_REQUIRE(x8 != nullptr && scale_inv != nullptr && weights != nullptr && weight_scaled != nullptr,
              "dsa_quant_rowwise_e4m3_weights: null pointer");
  DSA_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)x8 % 8) == 0, "dsa_quant_rowwise_e4m3_weights: misaligned pointer");
  if (rows == 0) return DSA_OK;
  int64_t blocks = (rows + 15) / 16;
  DSA_REQUIRE(blocks < (1ll << 31), "dsa_quant_rowwise_e4m3_weights: too many rows");
  if (rotate)
    rotate_quant128_kernel<<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(
        (const uint4*)x, (uint2*)x8, scale_inv, nullptr, rows, eps, pow2, weights, factor, weight_scaled);
  else
    quant128_kernel<<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>(
        (const uint4*)x, (uint2*)x8, scale_inv, rows, eps, pow2, weights, factor, weight_scaled);
  DSA_CHECK_LAUNCH("dsa_quant_rowwise_e4m3_weights");
  return DSA_OK;
}

extern "C" int dsa_indexer_front_e4m3(const void* x, int64_t rows, int cols, int rows_per_token, const float* ln_weight,
                                      const float* ln_bias, float ln_eps, const void* cos, const void* sin,
                                      int cos_sin_f32, int pairing, const int32_t* positions, int batch, int rotate,
                                      void* x8, float* scale_inv, void* y, float eps, int pow2, const float* weights,
                                      float factor, float* weight_scaled, void* stream) {
  DSA_REQUIRE(cols == 128, "dsa_indexer_front_e4m3: only rows of 128 elements are supported, got %d", cols);
  DSA_REQUIRE(rows >= 0 && rows_per_token > 0 && batch > 0, "dsa_indexer_front_e4m3: bad row counts");
  DSA_REQUIRE(pairing >= -1 && pairing <= 1, "dsa_indexer_front_e4m3: pairing must be -1 (no rotary part), 0 or 1");
  DSA_REQUIRE(pairing < 0 || (cos != nullptr && sin != nullptr), "dsa_indexer_front_e4m3: rotary part without cos / sin");
  DSA_REQUIRE((ln_weight == nullptr) == (ln_bias == nullptr), "dsa_indexer_front_e4m3: LayerNorm needs weight and bias");
  DSA_REQUIRE(x8 != nullptr || y != nullptr, "dsa_indexer_front_e4m3: no output requested");
  DSA_REQUIRE(x8 == nullptr || scale_inv != nullptr, "dsa_indexer_front_e4m3: payload without scales");
  DSA_REQUIRE((weights == nullptr) == (weight_scaled == nullptr) && (weights == nullptr || x8 != nullptr),
              "dsa_indexer_front_e4m3: weights and weight_scaled come together, with the payload");
  DSA_REQUIRE(((uintptr_t)x % 16) == 0 && ((uintptr_t)x8 % 8) == 0 && ((uintptr_t)y % 16) == 0 &&
              ((uintptr_t)ln_weight % 16) == 0 && ((uintptr_t)ln_bias % 16) == 0 && ((uintptr_t)cos % 16) == 0 &&
              ((uintptr_t)sin % 16) == 0, "dsa_indexer_front_e4m3: misaligned pointer");
  if (rows == 0) return DSA_OK;
  const int64_t blocks = (rows + 15) / 16;
  DSA_REQUIRE(blocks < (1ll << 31), "dsa_indexer_front_e4m3: too many rows");
#define DSA_FRONT_LAUNCH(LN, P) indexer_front128_kernel<LN, P><<<dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream>>>( \
      (const uint4*)x, rows, rows_per_token, ln_weight, ln_bias, ln_eps, cos, sin, cos_sin_f32, positions, batch, rotate, \
      (uint2*)x8, scale_inv, (uint4*)y, eps, pow2, weights, factor, weight_scaled)
  if (ln_weight) {
    if (pairing < 0) DSA_FRONT_LAUNCH(true, -1); else if (pairing == 0) DSA_FRONT_LAUNCH(true, 0); else DSA_FRONT_LAUNCH(true, 1);
  } else {
    if (pairing < 0) DSA_FRONT_LAUNCH(false, -1); else if (pairing == 0) DSA_FRONT_LAUNCH(false, 0); else DSA_FRONT_LAUNCH(false, 1);
  }
#undef DSA_FRONT_LAUNCH
  DSA_CHECK_LAUNCH("dsa_indexer_front_e4m3");
  return DSA_OK;
}
