// Key-sorted order of the valid (query, slot) pairs of a block of queries, built with integer
// work only (bitmap key x query, row-wise prefix popcounts, exclusive scan over keys), so it is
// identical from run to run.  Used by the deterministic scatter-accumulations of the backward
// kernels: pair (q, slot) with key v gets row  start[v] + #{q' < q : q' selects v}.
// Ids within one query row must be distinct (any top-k guarantees it): a repeated id has one bit and
// one row like any other, so one of its contributions would be lost.  The first kernel notices a
// repeated id (the bit it sets is set already) and raises *dup_flag; the callers' last kernels then
// fill their outputs with NaN instead of returning sums that silently miss a term.
#pragma once
#include "dsa_common.h"

namespace order {

static __global__ void zero_u32_kernel(unsigned* __restrict__ p, size_t n) {
  for (size_t e = (size_t)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (size_t)gridDim.x * blockDim.x) p[e] = 0u;
}

// bitmap[key][w] bit b  <=>  local query 32w + b selects key.
// Built without global atomics, in two steps.  (1) One workgroup per query sets the query's bits
// over the keys in LDS and writes them out as one row of qmap[query][key / 32] (Wk words).
// (2) A transpose of the bit matrix: a wave loads the words of 64 consecutive queries for one key
// word and turns bit b of all lanes into the 64-bit mask of key 32*kw + b with one ballot; the
// masks of 4 such query groups are combined through LDS so that every key receives 32 contiguous
// bytes.
static __global__ __launch_bounds__(256) void qmap_kernel(const int* __restrict__ ids, int q0, int cnt, int K, int Skv,
                                                          int q_start, unsigned* __restrict__ qmap, int Wk,
                                                          int* __restrict__ sorted, int* __restrict__ dup_flag) {
  extern __shared__ unsigned qbits[];        // Wk words; with `sorted`, Wk more for the prefix counts and K for the list
  __shared__ int wave_tot[4];
  const int ql = blockIdx.x;
  for (int w = threadIdx.x; w < Wk; w += 256) qbits[w] = 0u;
  __syncthreads();
  for (int t0 = threadIdx.x; t0 < K; t0 += 8 * 256) {
    int v[8];
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = t0 + i * 256 < K ? ids[(size_t)(q0 + ql) * K + t0 + i * 256] : -1;
#pragma unroll
    for (int i = 0; i < 8; i++)
      if (v[i] >= 0 && v[i] < Skv && v[i] <= q_start + q0 + ql) {
        const unsigned bit = 1u << (v[i] & 31);
        if (atomicOr(&qbits[v[i] >> 5], bit) & bit) *dup_flag = 1;      // every writer stores the same value
      }
  }
  __syncthreads();
  for (int w = threadIdx.x; w < Wk; w += 256) qmap[(size_t)ql * Wk + w] = qbits[w];
  if (sorted == nullptr) return;
  // The query's valid ids in ascending order, -1 after them: id v goes to position (set bits below v).
  // Thread t counts the words [t * per, (t + 1) * per); an exclusive scan over the threads gives each
  // thread its base, from which it writes the per-word prefix counts.
  unsigned* pre = qbits + Wk;
  const int per = (Wk + 255) / 256;
  const int w0 = threadIdx.x * per;
  int mine = 0;
  for (int w = w0; w < w0 + per && w < Wk; w++) mine += __popc(qbits[w]);
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int inc = mine;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) { int n = __shfl_up(inc, o, 64); if (lane >= o) inc += n; }
  if (lane == 63) wave_tot[wave] = inc;
  __syncthreads();
  int base = inc - mine;
  for (int w = 0; w < wave; w++) base += wave_tot[w];
  const int total = wave_tot[0] + wave_tot[1] + wave_tot[2] + wave_tot[3];
  for (int w = w0; w < w0 + per && w < Wk; w++) { pre[w] = (unsigned)base; base += __popc(qbits[w]); }
  __syncthreads();
  int* list = (int*)(pre + Wk);              // K ints: the list is put together in LDS and written out in order
  for (int t = total + threadIdx.x; t < K; t += 256) list[t] = -1;
  for (int t = threadIdx.x; t < K; t += 256) {
    const int v = ids[(size_t)(q0 + ql) * K + t];
    if (v >= 0 && v < Skv && v <= q_start + q0 + ql)
      list[pre[v >> 5] + __popc(qbits[v >> 5] & ((1u << (v & 31)) - 1u))] = v;
  }
  __syncthreads();
  int* row = sorted + (size_t)ql * K;
  for (int t = threadIdx.x; t < K; t += 256) row[t] = list[t];
}

// grid (ceil(cnt / 256), Wk); workgroup = 4 waves = 256 queries of one key word
static __global__ __launch_bounds__(256) void bm_transpose_kernel(const unsigned* __restrict__ qmap, int cnt, int Skv, int Wk,
                                                                  unsigned* __restrict__ bitmap, int W) {
  __shared__ unsigned long long mask_s[32][4];
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int kw = blockIdx.y;
  const int ql = blockIdx.x * 256 + threadIdx.x;
  const unsigned word = ql < cnt ? qmap[(size_t)ql * Wk + kw] : 0u;
#pragma unroll
  for (int b = 0; b < 32; b++) {
    const unsigned long long m = __ballot((word >> b) & 1u);
    if (lane == b) mask_s[b][wave] = m;
  }
  __syncthreads();
  // thread t < 256: key bit t / 8, 32-bit piece t % 8 of the 256 queries of this workgroup
  const int b = threadIdx.x >> 3, piece = threadIdx.x & 7;
  const int key = kw * 32 + b;
  const int w = blockIdx.x * 8 + piece;
  if (key < Skv && w < W) bitmap[(size_t)key * W + w] = ((const unsigned*)&mask_s[b][0])[piece];
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
static __global__ void rank_kernel(const int* __restrict__ ids, int row0, int q0, int cnt, int K, int Skv, int q_start,
                            const unsigned* __restrict__ bitmap, const unsigned* __restrict__ prefix,
                            const int* __restrict__ start, int W, int* __restrict__ dst) {
  // blockIdx.y walks the queries, blockIdx.x the slots of one query in steps of the block size
  for (int ql = blockIdx.y; ql < cnt; ql += gridDim.y) {
    const int slot = blockIdx.x * blockDim.x + threadIdx.x;
    if (slot >= K) continue;
    const int v = ids[(size_t)(row0 + ql) * K + slot];      // row0: row of local query 0 in the id array handed in
    int d = -1;
    if (v >= 0 && v < Skv && v <= q_start + q0 + ql) {
      const size_t wi = (size_t)v * W + (ql >> 5);
      d = start[v] + (int)prefix[wi] + __popc(bitmap[wi] & ((1u << (ql & 31)) - 1u));
    }
    dst[(size_t)ql * K + slot] = d;
  }
}


// Launches the five kernels above for queries [q0, q0 + cnt).  A slot counts when its id v is in
// [0, Skv) and v <= q_start + (query index); pass a huge q_start to accept every id in range.
// With `sorted` ([cnt][K] ints) the first kernel also writes every query's valid ids in ascending
// order (-1 after them) and dst refers to the slots of that list: a caller that is free to choose
// its slot order uses the list instead of ids, which makes concurrently running queries gather
// neighbouring key rows at the same time (the rows then hit in the L2 of the XCD).
// The prefix buffer doubles as the scratch of step (1) (cnt * ceil(Skv / 32) words; it is rewritten by
// the prefix pass afterwards): size it with prefix_words().
inline size_t prefix_words(int chunk, int Skv) {
  const size_t W = (size_t)(chunk + 31) / 32, Wk = (size_t)(Skv + 31) / 32;
  return (size_t)Skv * W > (size_t)chunk * Wk ? (size_t)Skv * W : (size_t)chunk * Wk;
}
// The first kernel keeps one bit per key in LDS: the largest key count the builder takes
constexpr int MAX_KEYS = 150 * 1024 * 8;
// LDS of the first kernel with the sorted list: bitmap and prefix counts over all keys plus the list
inline bool sorted_list_fits(int Skv, int K) {
  return (size_t)((Skv + 31) / 32) * 8 + (size_t)K * 4 <= (size_t)150 * 1024;
}
// dup_flag: one int the caller has cleared (clear_flag) before the first block of queries of a call.
inline void clear_flag(int* dup_flag, hipStream_t st) { zero_u32_kernel<<<dim3(1), dim3(64), 0, st>>>((unsigned*)dup_flag, 1); }
inline void build(const int* ids, int q0, int cnt, int K, int Skv, int q_start, unsigned* bitmap, unsigned* prefix,
                  int* count, int* start, int* dst, int W, hipStream_t st, int* dup_flag, int* sorted = nullptr) {
  const int Wk = (Skv + 31) / 32;
  unsigned* qmap = prefix;
  const size_t lds = (size_t)Wk * 4 * (sorted ? 2 : 1) + (sorted ? (size_t)K * 4 : 0);
  if (lds > 48 * 1024)
    (void)hipFuncSetAttribute((const void*)qmap_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
  qmap_kernel<<<dim3(cnt), dim3(256), lds, st>>>(ids, q0, cnt, K, Skv, q_start, qmap, Wk, sorted, dup_flag);
  // every word of the bitmap is written (zeros beyond the last query), so no clearing pass is needed
  bm_transpose_kernel<<<dim3((W + 7) / 8, Wk), dim3(256), 0, st>>>(qmap, cnt, Skv, Wk, bitmap, W);
  bm_prefix_kernel<<<dim3((Skv + 3) / 4), dim3(256), 0, st>>>(bitmap, prefix, count, Skv, W);
  key_scan_kernel<<<dim3(1), dim3(1024), 0, st>>>(count, start, Skv);
  // with `sorted` (rows of the block's queries, [cnt][K]) the ranks are those of the sorted slots
  rank_kernel<<<dim3((K + 255) / 256, cnt < 32768 ? cnt : 32768), dim3(256), 0, st>>>(sorted ? sorted : ids, sorted ? 0 : q0, q0, cnt,
                                                                                     K, Skv, q_start, bitmap, prefix, start, W, dst);
}

}  // namespace order
