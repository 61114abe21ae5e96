// Key-sorted order of the valid (query, slot) pairs of a block of queries, built with integer
// work only (bitmap key x query, row-wise prefix popcounts, exclusive scan over keys), so it is
// identical from run to run.  Used by the deterministic scatter-accumulations of the backward
// kernels: pair (q, slot) with key v gets row  start[v] + #{q' < q : q' selects v}.
// Ids within one query row must be distinct (any top-k guarantees it).
#pragma once
#include "dsa_common.h"

namespace order {

static __global__ void zero_u32_kernel(unsigned* __restrict__ p, size_t n) {
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) p[e] = 0u;
}

// bitmap[key][w] bit b  <=>  local query 32w + b selects key
static __global__ void bm_set_kernel(const int* __restrict__ ids, int q0, int cnt, int K, int Skv, int q_start,
                              unsigned* __restrict__ bitmap, int W) {
  const size_t n = (size_t)cnt * K;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) {
    const int ql = (int)(e / K);
    const int v = ids[(size_t)(q0 + ql) * K + (e % K)];
    if (v >= 0 && v < Skv && v <= q_start + q0 + ql) atomicOr(&bitmap[(size_t)v * W + (ql >> 5)], 1u << (ql & 31));
  }
}

// prefix[key][w] = number of set bits in words < w; count[key] = total.  One wave per key.
static __global__ __launch_bounds__(256) void bm_prefix_kernel(const unsigned* __restrict__ bitmap, unsigned* __restrict__ prefix,
                                                        int* __restrict__ count, int Skv, int W) {
  const int lane = threadIdx.x & 63;
  const int key = blockIdx.x * 4 + (threadIdx.x >> 6);
  if (key >= Skv) return;
  int run = 0;
  for (int w0 = 0; w0 < W; w0 += 64) {
    const int w = w0 + lane;
    const int c = w < W ? __popc(bitmap[(size_t)key * W + w]) : 0;
    int inc = c;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) { int n = __shfl_up(inc, o, 64); if (lane >= o) inc += n; }
    if (w < W) prefix[(size_t)key * W + w] = (unsigned)(run + inc - c);
    run += __shfl(inc, 63, 64);
  }
  if (lane == 0) count[key] = run;
}

// start[key] = exclusive prefix sum of count (single workgroup; Skv is at most a few 10^5)
static __global__ __launch_bounds__(1024) void key_scan_kernel(const int* __restrict__ count, int* __restrict__ start, int Skv) {
  __shared__ int wsum[16];
  __shared__ int carry_s;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) carry_s = 0;
  __syncthreads();
  for (int base = 0; base < Skv; base += 1024) {
    const int k = base + tid;
    const int c = k < Skv ? count[k] : 0;
    int inc = c;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) { int n = __shfl_up(inc, o, 64); if (lane >= o) inc += n; }
    if (lane == 63) wsum[wave] = inc;
    __syncthreads();
    int before = carry_s;
    for (int w = 0; w < wave; w++) before += wsum[w];
    if (k < Skv) start[k] = before + inc - c;
    __syncthreads();
    if (tid == 1023) carry_s = before + inc;
    __syncthreads();
  }
  if (tid == 0) start[Skv] = carry_s;
}

// dst[ql][slot] = row of the pair in key-sorted order (-1 for invalid slots)
static __global__ void rank_kernel(const int* __restrict__ ids, int q0, int cnt, int K, int Skv, int q_start,
                            const unsigned* __restrict__ bitmap, const unsigned* __restrict__ prefix,
                            const int* __restrict__ start, int W, int* __restrict__ dst) {
  const size_t n = (size_t)cnt * K;
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) {
    const int ql = (int)(e / K);
    const int v = ids[(size_t)(q0 + ql) * K + (e % K)];
    int d = -1;
    if (v >= 0 && v < Skv && v <= q_start + q0 + ql) {
      const size_t wi = (size_t)v * W + (ql >> 5);
      d = start[v] + (int)prefix[wi] + __popc(bitmap[wi] & ((1u << (ql & 31)) - 1u));
    }
    dst[e] = d;
  }
}


// Launches the five kernels above for queries [q0, q0 + cnt).  A slot counts when its id v is in
// [0, Skv) and v <= q_start + (query index); pass a huge q_start to accept every id in range.
inline void build(const int* ids, int q0, int cnt, int K, int Skv, int q_start, unsigned* bitmap, unsigned* prefix,
                  int* count, int* start, int* dst, int W, hipStream_t st) {
  zero_u32_kernel<<<dim3(1024), dim3(256), 0, st>>>(bitmap, (size_t)Skv * W);
  bm_set_kernel<<<dim3(2048), dim3(256), 0, st>>>(ids, q0, cnt, K, Skv, q_start, bitmap, W);
  bm_prefix_kernel<<<dim3((Skv + 3) / 4), dim3(256), 0, st>>>(bitmap, prefix, count, Skv, W);
  key_scan_kernel<<<dim3(1), dim3(1024), 0, st>>>(count, start, Skv);
  rank_kernel<<<dim3(2048), dim3(256), 0, st>>>(ids, q0, cnt, K, Skv, q_start, bitmap, prefix, start, W, dst);
}

}  // namespace order
