// KL loss of the indexer against the attention distribution, with its gradient, in one pass (gfx950).
//
// Per query row, over the K selected slots:
//   pred = softmax(score)        u = target + eps
//   loss_row = sum_t u_t (log u_t - log(pred_t + eps))                       (F.kl_div(log(pred + eps), u, "sum"))
//   grad_t   = d loss_row / d score_t = pred_t (sum_j w_j pred_j - w_t),     w_t = u_t / (pred_t + eps)
// One workgroup per row; the row's scores and targets stay in registers between the three reductions
// (maximum, normaliser, loss and sum_j w_j pred_j), so each array crosses HBM once and the gradient is
// written once.  A padded slot (score -inf, target 0) has pred = 0, contributes eps (log eps - log eps) = 0
// to the loss and gets gradient 0.  HBM-bound: 12 bytes per slot.
#include "dsa_common.h"

namespace {

constexpr int BLOCK = 256;

// sums (or maxima) over the workgroup; every thread gets the result.  `scratch` holds 8 floats.
__device__ __forceinline__ float block_max(float v, float* scratch) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, 64));
  __syncthreads();                                   // the previous reduction's reads are done
  if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = v;
  __syncthreads();
  return fmaxf(fmaxf(scratch[0], scratch[1]), fmaxf(scratch[2], scratch[3]));
}
__device__ __forceinline__ void block_sum2(float& a, float& b, float* scratch) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) { a += __shfl_xor(a, o, 64); b += __shfl_xor(b, o, 64); }
  __syncthreads();
  if ((threadIdx.x & 63) == 0) { scratch[threadIdx.x >> 6] = a; scratch[4 + (threadIdx.x >> 6)] = b; }
  __syncthreads();
  a = (scratch[0] + scratch[1]) + (scratch[2] + scratch[3]);
  b = (scratch[4] + scratch[5]) + (scratch[6] + scratch[7]);
}

template <int NE>   // slots per thread: K <= NE * BLOCK
__global__ __launch_bounds__(BLOCK) void kl_loss_kernel(const float* __restrict__ scores, int64_t ld_s,
                                                        const float* __restrict__ target, int64_t ld_t, int K, float eps,
                                                        float* __restrict__ row_loss, float* __restrict__ grad) {
  __shared__ float scratch[8];
  const int tid = threadIdx.x;
  const int64_t row = blockIdx.x;
  const float* sp = scores + row * ld_s;
  const float* tp = target + row * ld_t;
  float s[NE], u[NE];
  float mx = -INFINITY;
#pragma unroll
  for (int i = 0; i < NE; i++) {
    const int t = tid + BLOCK * i;
    s[i] = t < K ? sp[t] : -INFINITY;
    u[i] = (t < K ? tp[t] : 0.f) + eps;
    mx = fmaxf(mx, s[i]);
  }
  mx = block_max(mx, scratch);
  float z = 0.f, unused = 0.f;
#pragma unroll
  for (int i = 0; i < NE; i++) { s[i] = expf(s[i] - mx); z += s[i]; }     // a row of -inf only: NaN, as torch.softmax
  block_sum2(z, unused, scratch);
  const float inv = 1.0f / z;
  float loss = 0.f, inner = 0.f;
#pragma unroll
  for (int i = 0; i < NE; i++) {
    const int t = tid + BLOCK * i;
    const float p = s[i] * inv;
    const float w = u[i] / (p + eps);
    if (t < K) {
      loss += u[i] * (logf(u[i]) - logf(p + eps));
      inner += w * p;
    }
    s[i] = p;
    u[i] = w;
  }
  block_sum2(loss, inner, scratch);
#pragma unroll
  for (int i = 0; i < NE; i++) {
    const int t = tid + BLOCK * i;
    if (t < K) grad[row * K + t] = s[i] * (inner - u[i]);
  }
  if (tid == 0) row_loss[row] = loss;
}

}  // namespace

extern "C" int dsa_indexer_kl_loss(const float* scores, int64_t ld_s, const float* target, int64_t ld_t, int S, int K,
                                   float eps, float* row_loss, float* grad, void* stream) {
  DSA_REQUIRE(S >= 0 && K > 0 && K <= 32 * BLOCK, "dsa_indexer_kl_loss: K must lie in [1, %d], got %d", 32 * BLOCK, K);
  DSA_REQUIRE(ld_s >= K && ld_t >= K, "dsa_indexer_kl_loss: row strides %lld / %lld below K = %d", (long long)ld_s,
              (long long)ld_t, K);
  if (S == 0) return DSA_OK;
  hipStream_t st = (hipStream_t)stream;
  if (K <= 8 * BLOCK) kl_loss_kernel<8><<<dim3(S), dim3(BLOCK), 0, st>>>(scores, ld_s, target, ld_t, K, eps, row_loss, grad);
  else kl_loss_kernel<32><<<dim3(S), dim3(BLOCK), 0, st>>>(scores, ld_s, target, ld_t, K, eps, row_loss, grad);
  DSA_CHECK_LAUNCH("dsa_indexer_kl_loss");
  return DSA_OK;
}
