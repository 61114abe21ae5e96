// Head-averaged softmax over the selected slots: target[i,t] = mean_h softmax_t(p_out[i,h,:] * c).
// HBM-bound: reads H*K logits per query once.  One workgroup per query; each wave takes heads
// w, w+4, ...; a head's K logits live in registers, so p_out is read exactly once.  Two variants:
// 16-byte loads when the layout allows it, element loads otherwise (the same arithmetic; the partial
// sums of a head are grouped differently, so results agree to fp32 rounding, not bit for bit).
// exp2 is the bare hardware instruction (the arguments are <= 0; results below 2^-126 flush to zero):
// the library routine's range handling costs four more instructions per logit, and this kernel is
// bound by them.
#include "dsa_common.h"

namespace {

constexpr int MAXV = 64;   // slots per lane: supports K <= 4096

template <bool F32>
__device__ __forceinline__ float load_logit(const void* p, int64_t off) {
  if (F32) return ((const float*)p)[off];
  return bf16_bits_to_f32(((const unsigned short*)p)[off]);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, 64);
  return v;
}

template <bool F32, int NV>
__global__ __launch_bounds__(256) void attn_dist_kernel(const void* __restrict__ p_out, int H, int K,
                                                        int64_t ld_s, int64_t ld_h, float c2,
                                                        float* __restrict__ target) {
  extern __shared__ float acc_s[];            // [4 waves][K]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t i = blockIdx.x;
  float acc[NV];
#pragma unroll
  for (int v = 0; v < NV; v++) acc[v] = 0.f;
  for (int h = wave; h < H; h += 4) {
    const int64_t base = i * ld_s + h * ld_h;
    float z[NV];
    float mx = -INFINITY;
#pragma unroll
    for (int v = 0; v < NV; v++) {
      int t = v * 64 + lane;
      z[v] = t < K ? load_logit<F32>(p_out, base + t) * c2 : -INFINITY;
      mx = fmaxf(mx, z[v]);
    }
    mx = wave_max(mx);
    if (mx == -INFINITY) continue;            // head with no valid slot contributes nothing
    float sum = 0.f;
#pragma unroll
    for (int v = 0; v < NV; v++) { z[v] = __builtin_amdgcn_exp2f(z[v] - mx); sum += z[v]; }
    sum = wave_sum(sum);
    float inv = 1.0f / sum;
#pragma unroll
    for (int v = 0; v < NV; v++) acc[v] += z[v] * inv;
  }
#pragma unroll
  for (int v = 0; v < NV; v++) { int t = v * 64 + lane; if (t < K) acc_s[wave * K + t] = acc[v]; }
  __syncthreads();
  const float invh = 1.0f / (float)H;
  for (int t = threadIdx.x; t < K; t += 256)
    target[i * K + t] = ((acc_s[t] + acc_s[K + t]) + (acc_s[2 * K + t] + acc_s[3 * K + t])) * invh;
}

// The same with 16-byte loads: lane l of a wave owns slots 8 (64 v + l) .. +7 of every head.  Needs
// K, the strides and the base address to be multiples of 8 elements, and a positive scale (the row
// maximum is taken on the raw logits).
template <bool F32, int NC>
__global__ __launch_bounds__(256) void attn_dist_vec_kernel(const void* __restrict__ p_out, int H, int K,
                                                            int64_t ld_s, int64_t ld_h, float c2,
                                                            float* __restrict__ target) {
  extern __shared__ float acc_s[];            // [4 waves][K]
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int64_t i = blockIdx.x;
  float acc[NC][8];
#pragma unroll
  for (int v = 0; v < NC; v++)
#pragma unroll
    for (int e = 0; e < 8; e++) acc[v][e] = 0.f;
  // raw 16-byte pieces of one head; the next head's are requested before this head's arithmetic
  struct Raw { uint4 a[NC]; uint4 b[NC]; };
  auto fetch = [&](int h, Raw& r) {
    const int64_t base = i * ld_s + h * ld_h;
#pragma unroll
    for (int v = 0; v < NC; v++) {
      const int t = 8 * (v * 64 + lane);
      if (t < K && h < H) {
        if (F32) {
          r.a[v] = *(const uint4*)((const float*)p_out + base + t);
          r.b[v] = *(const uint4*)((const float*)p_out + base + t + 4);
        } else {
          r.a[v] = *(const uint4*)((const unsigned short*)p_out + base + t);
        }
      }
    }
  };
  // one head: its softmax numerators, their sum, and the accumulation of the normalised values
  auto head = [&](const Raw& cur) {
    float z[NC][8];
    float mx = -INFINITY;
#pragma unroll
    for (int v = 0; v < NC; v++) {
      const int t = 8 * (v * 64 + lane);
      if (t < K) {
        if (F32) {
          const unsigned w[8] = {cur.a[v].x, cur.a[v].y, cur.a[v].z, cur.a[v].w, cur.b[v].x, cur.b[v].y, cur.b[v].z, cur.b[v].w};
#pragma unroll
          for (int e = 0; e < 8; e++) z[v][e] = __builtin_bit_cast(float, w[e]);
        } else {
          const unsigned w[4] = {cur.a[v].x, cur.a[v].y, cur.a[v].z, cur.a[v].w};
#pragma unroll
          for (int e = 0; e < 4; e++) {
            z[v][2 * e] = __builtin_bit_cast(float, w[e] << 16);
            z[v][2 * e + 1] = __builtin_bit_cast(float, w[e] & 0xffff0000u);
          }
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; e++) z[v][e] = -INFINITY;
      }
#pragma unroll
      for (int e = 0; e < 8; e++) mx = fmaxf(mx, z[v][e]);
    }
    mx = wave_max(mx);
    if (mx == -INFINITY) return;              // head with no valid slot contributes nothing
    // the (positive) scale enters through one fused multiply-add per logit: exp2(z c2 - max(z) c2)
    const float off = -mx * c2;
    float sum = 0.f;
#pragma unroll
    for (int v = 0; v < NC; v++)
#pragma unroll
      for (int e = 0; e < 8; e++) { z[v][e] = __builtin_amdgcn_exp2f(fmaf(z[v][e], c2, off)); sum += z[v][e]; }
    sum = wave_sum(sum);
    const float inv = 1.0f / sum;
#pragma unroll
    for (int v = 0; v < NC; v++)
#pragma unroll
      for (int e = 0; e < 8; e++) acc[v][e] += z[v][e] * inv;
  };
  // two buffers take turns (no register copies): while one head is worked on, the next is on its way
  Raw r0, r1;
  fetch(wave, r0);
  for (int h = wave; h < H; h += 8) {
    fetch(h + 4, r1);
    head(r0);
    if (h + 4 < H) {
      fetch(h + 8, r0);
      head(r1);
    }
  }
#pragma unroll
  for (int v = 0; v < NC; v++) {
    const int t = 8 * (v * 64 + lane);
    if (t < K) {
      *(f32x4*)(acc_s + wave * K + t) = f32x4{acc[v][0], acc[v][1], acc[v][2], acc[v][3]};
      *(f32x4*)(acc_s + wave * K + t + 4) = f32x4{acc[v][4], acc[v][5], acc[v][6], acc[v][7]};
    }
  }
  __syncthreads();
  const float invh = 1.0f / (float)H;
  for (int t = threadIdx.x; t < K; t += 256)
    target[i * K + t] = ((acc_s[t] + acc_s[K + t]) + (acc_s[2 * K + t] + acc_s[3 * K + t])) * invh;
}

template <bool F32>
int launch(const void* p_out, int S, int H, int K, int64_t ld_s, int64_t ld_h, float sm_scale, float* target,
           hipStream_t st) {
  const float c2 = sm_scale * 1.4426950408889634f;
  size_t smem = (size_t)4 * K * sizeof(float);
  const bool vec = K % 8 == 0 && ld_s % 8 == 0 && ld_h % 8 == 0 && ((uintptr_t)p_out % 32) == 0 && c2 > 0.f;
  if (vec) {
    const int nc = (K + 511) / 512;
#define DSA_ADV_CASE(N) \
    if (nc <= N) { attn_dist_vec_kernel<F32, N><<<dim3(S), dim3(256), smem, st>>>(p_out, H, K, ld_s, ld_h, c2, target); return 0; }
    DSA_ADV_CASE(1) DSA_ADV_CASE(2) DSA_ADV_CASE(4) DSA_ADV_CASE(8)
#undef DSA_ADV_CASE
  }
  int nv = (K + 63) / 64;
#define DSA_AD_CASE(N) \
  if (nv <= N) { attn_dist_kernel<F32, N><<<dim3(S), dim3(256), smem, st>>>(p_out, H, K, ld_s, ld_h, c2, target); return 0; }
  DSA_AD_CASE(1) DSA_AD_CASE(2) DSA_AD_CASE(4) DSA_AD_CASE(8) DSA_AD_CASE(16) DSA_AD_CASE(32) DSA_AD_CASE(64)
#undef DSA_AD_CASE
  return -1;
}

}  // namespace

extern "C" int dsa_attn_dist(const void* p_out, int p_out_f32, int S, int H, int K, int64_t ld_s, int64_t ld_h,
                             float sm_scale, float* target, void* stream) {
  DSA_REQUIRE(S >= 0 && H > 0 && K > 0, "dsa_attn_dist: bad shape S=%d H=%d K=%d", S, H, K);
  DSA_REQUIRE(K <= 64 * MAXV, "dsa_attn_dist: K=%d exceeds the supported maximum %d", K, 64 * MAXV);
  DSA_REQUIRE(ld_h >= K && ld_s >= ld_h, "dsa_attn_dist: bad strides");
  if (S == 0) return DSA_OK;
  int rc = p_out_f32 ? launch<true>(p_out, S, H, K, ld_s, ld_h, sm_scale, target, (hipStream_t)stream)
                     : launch<false>(p_out, S, H, K, ld_s, ld_h, sm_scale, target, (hipStream_t)stream);
  DSA_REQUIRE(rc == 0, "dsa_attn_dist: unsupported K");
  DSA_CHECK_LAUNCH("dsa_attn_dist");
  return DSA_OK;
}
