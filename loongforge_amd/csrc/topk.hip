// Per-row top-k selection (radix select with the candidate histograms in LDS) for gfx950.
//
// One workgroup per row.  General path: the row's window is read once into LDS as order-preserving
// 32-bit keys (or re-read from global memory when it does not fit); three histogram passes
// (12 + 10 + 10 bits, most significant first) locate the k-th largest key exactly, a prefix-sum
// compaction then emits every key above it plus the first ties in ascending column order, so the
// result is deterministic; an optional sorting network orders the K outputs by descending score.
// Sorted rows whose values spread over a range take a single sweep instead (linear_select_sort*):
// a histogram over equal-width value bins, a counting-sort scatter and a rank inside each bin; rows
// of up to 8192 columns are held in registers for it, which leaves room for four workgroups per
// compute unit.  HBM-bound by design (4 bytes read per candidate, 8 bytes written per output slot);
// in practice the LDS atomics of the histogram and the scatter set the pace.
#include "dsa_common.h"

namespace {

constexpr int BLOCK = 256;
constexpr int NW = BLOCK / 64;
constexpr int HBINS = 4096;

__device__ __forceinline__ unsigned f2key(float f) {       // larger float <-> larger unsigned
  unsigned u = __builtin_bit_cast(unsigned, f);
  return (u & 0x80000000u) ? ~u : (u | 0x80000000u);
}
__device__ __forceinline__ float key2f(unsigned k) {
  unsigned u = (k & 0x80000000u) ? (k & 0x7fffffffu) : ~k;
  return __builtin_bit_cast(float, u);
}

// exclusive prefix sum over the block (thread order), also returns the block total
__device__ __forceinline__ int block_exscan(int v, int* scratch, int& total) {
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int inc = v;
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    int n = __shfl_up(inc, o, 64);
    if (lane >= o) inc += n;
  }
  __syncthreads();
  if (lane == 63) scratch[wave] = inc;
  __syncthreads();
  int base = 0, tot = 0;
#pragma unroll
  for (int w = 0; w < NW; w++) { int s = scratch[w]; if (w < wave) base += s; tot += s; }
  total = tot;
  return base + inc - v;
}

struct Pick { int bin; int above; };

// Finds, scanning bins from the highest down, the bin in which the running count reaches `need`.
// hist has nb bins (nb % BLOCK == 0).  Result: that bin and the number of keys in higher bins.
__device__ __forceinline__ Pick pick_bin(const int* hist, int nb, int need, int* scratch, int* res) {
  const int per = nb / BLOCK;
  const int hi = nb - 1 - (int)threadIdx.x * per;          // this thread owns bins hi, hi-1, ..., hi-per+1
  int local = 0;
  for (int b = 0; b < per; b++) local += hist[hi - b];
  int total;
  int before = block_exscan(local, scratch, total);
  if (before < need && before + local >= need) {
    int run = before;
    for (int b = 0; b < per; b++) {
      int c = hist[hi - b];
      if (run + c >= need) { res[0] = hi - b; res[1] = run; break; }
      run += c;
    }
  }
  __syncthreads();
  Pick p = {res[0], res[1]};
  __syncthreads();
  return p;
}

// Order of the sorted output: descending score, ascending id among equal scores (id -1 last).
__device__ __forceinline__ bool comes_first(float a, int ia, float b, int ib) {
  return (a > b) || (a == b && (unsigned)ia < (unsigned)ib);
}

// Bitonic sort of Kp2 = EPT * BLOCK (score, id) pairs held in LDS.  A pair becomes one 64-bit
// key whose unsigned order is the output order (descending score, then ascending id, id -1 last),
// so a compare-exchange is one 64-bit compare and two selects.  Thread t keeps
// elements [t*EPT, (t+1)*EPT) in registers: strides below EPT are register compare-exchanges,
// strides inside a wave's span exchange through LDS without a workgroup barrier (LDS operations
// of one wave complete in order), and only the strides that cross waves need barriers.  The
// exchange buffer holds element j of thread t at j * BLOCK + t, so every LDS access of a wave is
// bank-conflict free; the sorted elements go straight from registers to global memory.
__device__ __forceinline__ unsigned long long sort_key(float score, int id) {
  const unsigned bits = __builtin_bit_cast(unsigned, score + 0.0f);          // -0 -> +0
  const unsigned asc = bits ^ ((bits >> 31) ? 0xffffffffu : 0x80000000u);    // ascending with the score
  return ((unsigned long long)(~asc) << 32) | (unsigned)id;
}
__device__ __forceinline__ float sort_key_score(unsigned long long key) {
  const unsigned asc = ~(unsigned)(key >> 32);
  return __builtin_bit_cast(float, asc ^ ((asc >> 31) ? 0x80000000u : 0xffffffffu));
}

template <int EPT>
__device__ __forceinline__ void bitonic_regs(float* outv, int* outi, unsigned long long* xbuf, int Kp2, float* sv, int* si, int K) {
  const int tid = threadIdx.x;
  const int base = tid * EPT;
  unsigned long long key[EPT];
#pragma unroll
  for (int j = 0; j < EPT; j++) key[j] = sort_key(outv[base + j], outi[base + j]);
  __syncthreads();                             // the buffer is reused as the exchange buffer below
  for (int size = 2; size <= Kp2; size <<= 1) {
    for (int stride = size >> 1; stride > 0; stride >>= 1) {
      if (stride >= EPT) {
        const int pt = tid ^ (stride / EPT);
        const bool cross_wave = stride / EPT >= 64;
#pragma unroll
        for (int j = 0; j < EPT; j++) xbuf[j * BLOCK + tid] = key[j];
        if (cross_wave) __syncthreads(); else __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
        unsigned long long pk[EPT];
#pragma unroll
        for (int j = 0; j < EPT; j++) pk[j] = xbuf[j * BLOCK + pt];
        if (cross_wave) __syncthreads(); else __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
        // this lane keeps the smaller key when it holds the lower element of an ascending pair or
        // the upper element of a descending one (size > stride >= EPT: the same for all j)
        const bool keep_small = ((base & stride) == 0) == ((base & size) == 0);
#pragma unroll
        for (int j = 0; j < EPT; j++) key[j] = ((key[j] < pk[j]) == keep_small) ? key[j] : pk[j];
      } else {
#pragma unroll
        for (int st = EPT >> 1; st > 0; st >>= 1) {
          if (st != stride) continue;
#pragma unroll
          for (int j = 0; j < EPT; j++) {
            if (j & st) continue;
            const bool asc = ((base + j) & size) == 0;
            const unsigned long long x = key[j], y = key[j | st];
            const bool x_first = (x < y) == asc;
            key[j] = x_first ? x : y;
            key[j | st] = x_first ? y : x;
          }
        }
      }
    }
  }
#pragma unroll
  for (int j = 0; j < EPT; j++)
    if (base + j < K) { sv[base + j] = sort_key_score(key[j]); si[base + j] = (int)(unsigned)key[j]; }
}

// Sorted top-K of a staged row in one sweep, for rows whose finite values spread over a range:
// a histogram over HBINS equal-width value bins (bin 0 = largest values) finds the bin that holds
// the K-th largest value; every element of a better bin, plus all elements of that bin, is
// scattered into its bin's segment of an LDS buffer (a counting sort, segments in descending value
// order), and each scattered element then finds its final position by counting the elements of its
// own segment that precede it in the output order (descending score, ascending column).  Elements
// of the threshold bin that rank beyond the K-th place are dropped.  The result is exact and does
// not depend on the order in which the atomics land.  Returns false without writing anything when
// the row is unsuitable (no spread, or a crowded bin): the caller then takes the general path.
constexpr int LIN_SPARE = 960;               // extra buffer entries for the threshold bin's surplus
constexpr int REG_ROW = 8192 + 4 * 256;      // longest row (plus alignment slack) the register variant holds
constexpr int REG_ROW_BIG = 32768 + 4 * 256; // the same for the variant with twice the registers
constexpr int LIN_MAX_BIN = 256;             // largest segment ranked by pairwise counting

// Threshold bin of a filled histogram (thread t owns bins [PER t, PER t + PER)), then the segment
// starts written over the counts.  False when a bin is too crowded for the ranking step.
__device__ __forceinline__ bool lin_threshold(int* hist, int* scratch, int keff, int& tbin, int& above, int& c) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr int PER = HBINS / BLOCK;
  int cnt[PER], local = 0;
#pragma unroll
  for (int b4 = 0; b4 < PER; b4 += 4) {
    const int4 q4 = *(const int4*)(hist + tid * PER + b4);
    cnt[b4] = q4.x; cnt[b4 + 1] = q4.y; cnt[b4 + 2] = q4.z; cnt[b4 + 3] = q4.w;
  }
#pragma unroll
  for (int b = 0; b < PER; b++) local += cnt[b];
  int total;
  const int before = block_exscan(local, scratch, total);
  if (before < keff && before + local >= keff) {
    int run = before;
#pragma unroll
    for (int b = 0; b < PER; b++) {
      if (run < keff && run + cnt[b] >= keff) { scratch[8] = tid * PER + b; scratch[9] = run; scratch[10] = cnt[b]; }
      run += cnt[b];
    }
  }
  __syncthreads();
  tbin = scratch[8]; above = scratch[9]; c = scratch[10];
  int big = 0;
#pragma unroll
  for (int b = 0; b < PER; b++) if (tid * PER + b < tbin) big = max(big, cnt[b]);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) big = max(big, __shfl_xor(big, o, 64));
  __syncthreads();
  if (lane == 0) scratch[wave] = big;
  __syncthreads();
  big = max(max(scratch[0], scratch[1]), max(scratch[2], scratch[3]));
  if (big > LIN_MAX_BIN || c > LIN_SPARE) return false;
  {
    int run = before, st[PER];
#pragma unroll
    for (int b = 0; b < PER; b++) { st[b] = run; run += cnt[b]; }
#pragma unroll
    for (int b4 = 0; b4 < PER; b4 += 4) *(int4*)(hist + tid * PER + b4) = make_int4(st[b4], st[b4 + 1], st[b4 + 2], st[b4 + 3]);
  }
  __syncthreads();
  return true;
}

// Final position of every scattered element: hist[b] is the end of segment b by now.
template <class BinOf>
__device__ __forceinline__ void lin_rank(const unsigned long long* obuf, const int* hist, int filled, int keff, int K,
                                         int base_id, BinOf bin_of, float* sv, int* si) {
  const int tid = threadIdx.x;
  for (int p = tid; p < filled; p += BLOCK) {
    const unsigned long long key = obuf[p];
    const float v = sort_key_score(key);
    const int b = bin_of(v);
    const int start = b > 0 ? hist[b - 1] : 0, end = hist[b];
    int rank = 0;
    for (int j = start; j < end; j++) rank += obuf[j] < key;
    const int pos = start + rank;
    if (pos < keff) { sv[pos] = v; si[pos] = base_id + (int)(unsigned)key; }
  }
  for (int t = keff + tid; t < K; t += BLOCK) { sv[t] = -INFINITY; si[t] = -1; }
}

__device__ __forceinline__ bool linear_select_sort(const float* __restrict__ src, unsigned* keys, int n, int K, int base_id,
                                                   int* hist, int* scratch, unsigned long long* obuf, float* sv, int* si) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // ---- stage the row as keys; range of the finite values ---------------------------------------
  float mn = INFINITY, mx = -INFINITY;
  int nfin = 0;
  for (int e0 = tid; e0 < n; e0 += 8 * BLOCK) {   // eight loads in flight per thread
    float v[8];
#pragma unroll
    for (int i = 0; i < 8; i++) v[i] = e0 + i * BLOCK < n ? src[e0 + i * BLOCK] : -INFINITY;
#pragma unroll
    for (int i = 0; i < 8; i++) {
      if (e0 + i * BLOCK < n) keys[e0 + i * BLOCK] = f2key(v[i]);
      if (fabsf(v[i]) < INFINITY) { mn = fminf(mn, v[i]); mx = fmaxf(mx, v[i]); nfin++; }
      else if (!(v[i] < INFINITY)) mx = INFINITY;   // +inf or NaN: infinite span below, the general path takes the row
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, o, 64));
    mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    nfin += __shfl_xor(nfin, o, 64);
  }
  __syncthreads();
  if (lane == 0) { ((float*)scratch)[wave] = mn; ((float*)scratch)[4 + wave] = mx; scratch[8 + wave] = nfin; }
  __syncthreads();
  mn = fminf(fminf(((float*)scratch)[0], ((float*)scratch)[1]), fminf(((float*)scratch)[2], ((float*)scratch)[3]));
  mx = fmaxf(fmaxf(((float*)scratch)[4], ((float*)scratch)[5]), fmaxf(((float*)scratch)[6], ((float*)scratch)[7]));
  nfin = scratch[8] + scratch[9] + scratch[10] + scratch[11];
  __syncthreads();
  const float span = mx - mn;
  if (!(span > 0.f) || !(span < INFINITY)) return false;
  const int keff = min(K, nfin);
  const float scale = ((float)HBINS - 0.5f) / span;
  auto bin_of = [&](float v) { return min(HBINS - 1, (int)((mx - v) * scale)); };
  // ---- histogram ------------------------------------------------------------------------------
  for (int b = tid; b < HBINS; b += BLOCK) hist[b] = 0;
  __syncthreads();
  for (int e = tid; e < n; e += BLOCK) {
    const float v = key2f(keys[e]);
    if (fabsf(v) < INFINITY) atomicAdd(&hist[bin_of(v)], 1);
  }
  __syncthreads();
  int tbin, above, c;
  if (!lin_threshold(hist, scratch, keff, tbin, above, c)) return false;
  // ---- scatter ------------------------------------------------------------------------------------
  for (int e = tid; e < n; e += BLOCK) {
    const float v = key2f(keys[e]);
    if (fabsf(v) < INFINITY) {
      const int b = bin_of(v);
      if (b <= tbin) obuf[atomicAdd(&hist[b], 1)] = sort_key(v, e);
    }
  }
  __syncthreads();
  lin_rank(obuf, hist, above + c, keff, K, base_id, bin_of, sv, si);
  return true;
}

// The same for rows of at most 4 NV BLOCK elements, with the row held in registers instead of
// LDS: thread t owns the 16-byte chunks t, t + BLOCK, ... of the row counted from the 16-byte
// boundary at or below its first element, so the whole row is fetched by NV vector loads issued
// together and the workgroup needs only the histogram and the output buffer in LDS.  The row is
// positions [off, m) of that layout; chunk i (positions [4 BLOCK i, 4 BLOCK (i + 1))) is touched only
// while it holds any of them.
template <int NV>
__device__ __forceinline__ void load_row_regs(const float* __restrict__ src, int n, float (&v)[NV][4], int& off, int& m) {
  const int tid = threadIdx.x;
  off = (int)(((uintptr_t)src >> 2) & 3);                  // elements between that boundary and src
  const float* base = src - off;
  m = n + off;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    const int p = 4 * (tid + BLOCK * i);
    if (p >= off && p + 4 <= m) {
      const float4 x = *(const float4*)(base + p);
      v[i][0] = x.x; v[i][1] = x.y; v[i][2] = x.z; v[i][3] = x.w;
    } else {
#pragma unroll
      for (int j = 0; j < 4; j++) v[i][j] = (p + j >= off && p + j < m) ? base[p + j] : -INFINITY;
    }
  }
}

// min / max of three without the canonicalising v_max that fminf / fmaxf put in front of every operand
__device__ __forceinline__ float min3_raw(float a, float b, float c) {
  float r;
  asm("v_min3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}
__device__ __forceinline__ float max3_raw(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// The selection itself for rows whose values are all finite - the common case.  No per-element
// finiteness tests (an infinity shows in the row's minimum or maximum, a NaN in one unordered compare
// per two elements), min / max three at a time, bins without a clamp ((mx - x) scale < HBINS for every
// x in [mn, mx]), and chunks wholly inside the row need no position tests.  Returns 1 when the row is
// done, 0 when it is unsuitable (no spread, a crowded bin), -1 when it holds a non-finite value (the
// caller then runs the tolerant form below on the same registers).
template <int NV>
__device__ __forceinline__ int select_regs_finite(const float (&v)[NV][4], int off, int m, int K, int base_id, int* hist,
                                                  int* scratch, unsigned long long* obuf, float* sv, int* si) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  constexpr int CH = 4 * BLOCK;
  const int nch = (m + CH - 1) / CH;                        // chunks that hold any of the row
  auto chunk_full = [&](int i) { return (i > 0 || off == 0) && CH * (i + 1) <= m; };   // the same for all threads
  for (int b = tid; b < HBINS; b += BLOCK) hist[b] = 0;
  float mn = INFINITY, mx = -INFINITY;
  bool nan = false;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    if (i >= nch) continue;
    if (chunk_full(i)) {
      mn = min3_raw(mn, v[i][0], v[i][1]); mn = min3_raw(mn, v[i][2], v[i][3]);
      mx = max3_raw(mx, v[i][0], v[i][1]); mx = max3_raw(mx, v[i][2], v[i][3]);
      nan |= __builtin_isunordered(v[i][0], v[i][1]) | __builtin_isunordered(v[i][2], v[i][3]);
    } else {
      const int p = 4 * (tid + BLOCK * i);
#pragma unroll
      for (int j = 0; j < 4; j++)
        if (p + j >= off && p + j < m) {
          mn = min3_raw(mn, v[i][j], v[i][j]); mx = max3_raw(mx, v[i][j], v[i][j]);
          nan |= v[i][j] != v[i][j];
        }
    }
  }
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, o, 64));
    mx = fmaxf(mx, __shfl_xor(mx, o, 64));
  }
  const bool wave_nan = __ballot(nan) != 0ull;
  if (lane == 0) { ((float*)scratch)[wave] = mn; ((float*)scratch)[4 + wave] = mx; scratch[8 + wave] = wave_nan; }
  __syncthreads();
  mn = fminf(fminf(((float*)scratch)[0], ((float*)scratch)[1]), fminf(((float*)scratch)[2], ((float*)scratch)[3]));
  mx = fmaxf(fmaxf(((float*)scratch)[4], ((float*)scratch)[5]), fmaxf(((float*)scratch)[6], ((float*)scratch)[7]));
  const bool any_nan = (scratch[8] | scratch[9] | scratch[10] | scratch[11]) != 0;
  __syncthreads();
  if (any_nan || !(mn > -INFINITY) || !(mx < INFINITY)) return -1;
  const float span = mx - mn;
  if (!(span > 0.f) || !(span < INFINITY)) return 0;
  const int keff = min(K, m - off);
  const float scale = ((float)HBINS - 0.5f) / span;
  auto bin_of = [&](float x) { return (int)((mx - x) * scale); };
#pragma unroll
  for (int i = 0; i < NV; i++) {
    if (i >= nch) continue;
    if (chunk_full(i)) {
#pragma unroll
      for (int j = 0; j < 4; j++) atomicAdd(&hist[bin_of(v[i][j])], 1);
    } else {
      const int p = 4 * (tid + BLOCK * i);
#pragma unroll
      for (int j = 0; j < 4; j++)
        if (p + j >= off && p + j < m) atomicAdd(&hist[bin_of(v[i][j])], 1);
    }
  }
  __syncthreads();
  int tbin, above, c;
  if (!lin_threshold(hist, scratch, keff, tbin, above, c)) return 0;
#pragma unroll
  for (int i = 0; i < NV; i++) {
    if (i >= nch) continue;
    const int p = 4 * (tid + BLOCK * i);
    const bool full = chunk_full(i);
#pragma unroll
    for (int j = 0; j < 4; j++)
      if (full || (p + j >= off && p + j < m)) {
        const int b = bin_of(v[i][j]);
        if (b <= tbin) obuf[atomicAdd(&hist[b], 1)] = sort_key(v[i][j], p + j - off);
      }
  }
  __syncthreads();
  lin_rank(obuf, hist, above + c, keff, K, base_id, bin_of, sv, si);
  return 1;
}

// The tolerant form: values that are not finite (-inf marks a column that cannot be selected) are skipped
// one by one.
template <int NV>
__device__ __forceinline__ bool select_regs_tolerant(const float (&v)[NV][4], int off, int K, int base_id, int* hist,
                                                     int* scratch, unsigned long long* obuf, float* sv, int* si) {
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  for (int b = tid; b < HBINS; b += BLOCK) hist[b] = 0;
  float mn = INFINITY, mx = -INFINITY;
  int nfin = 0;
#pragma unroll
  for (int i = 0; i < NV; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
      if (fabsf(v[i][j]) < INFINITY) { mn = fminf(mn, v[i][j]); mx = fmaxf(mx, v[i][j]); nfin++; }
      else if (!(v[i][j] < INFINITY)) mx = INFINITY;   // +inf or NaN: the general path takes the row
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    mn = fminf(mn, __shfl_xor(mn, o, 64));
    mx = fmaxf(mx, __shfl_xor(mx, o, 64));
    nfin += __shfl_xor(nfin, o, 64);
  }
  if (lane == 0) { ((float*)scratch)[wave] = mn; ((float*)scratch)[4 + wave] = mx; scratch[8 + wave] = nfin; }
  __syncthreads();
  mn = fminf(fminf(((float*)scratch)[0], ((float*)scratch)[1]), fminf(((float*)scratch)[2], ((float*)scratch)[3]));
  mx = fmaxf(fmaxf(((float*)scratch)[4], ((float*)scratch)[5]), fmaxf(((float*)scratch)[6], ((float*)scratch)[7]));
  nfin = scratch[8] + scratch[9] + scratch[10] + scratch[11];
  __syncthreads();
  const float span = mx - mn;
  if (!(span > 0.f) || !(span < INFINITY)) return false;
  const int keff = min(K, nfin);
  const float scale = ((float)HBINS - 0.5f) / span;
  auto bin_of = [&](float x) { return min(HBINS - 1, (int)((mx - x) * scale)); };
#pragma unroll
  for (int i = 0; i < NV; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
      if (fabsf(v[i][j]) < INFINITY) atomicAdd(&hist[bin_of(v[i][j])], 1);
  __syncthreads();
  int tbin, above, c;
  if (!lin_threshold(hist, scratch, keff, tbin, above, c)) return false;
#pragma unroll
  for (int i = 0; i < NV; i++)
#pragma unroll
    for (int j = 0; j < 4; j++)
      if (fabsf(v[i][j]) < INFINITY) {
        const int b = bin_of(v[i][j]);
        if (b <= tbin) obuf[atomicAdd(&hist[b], 1)] = sort_key(v[i][j], 4 * (tid + BLOCK * i) + j - off);
      }
  __syncthreads();
  lin_rank(obuf, hist, above + c, keff, K, base_id, bin_of, sv, si);
  return true;
}

template <int NV>
__device__ __forceinline__ bool linear_select_sort_regs(const float* __restrict__ src, int n, int K, int base_id,
                                                        int* hist, int* scratch, unsigned long long* obuf, float* sv, int* si) {
  float v[NV][4];
  int off, m;
  load_row_regs<NV>(src, n, v, off, m);
  const int r = select_regs_finite<NV>(v, off, m, K, base_id, hist, scratch, obuf, sv, si);
  if (r >= 0) return r == 1;
  __syncthreads();
  return select_regs_tolerant<NV>(v, off, K, base_id, hist, scratch, obuf, sv, si);
}

// LEAN (sorted rows held in registers; implies !STAGED).  1: rows of up to REG_ROW elements, the kernel keeps to
// 128 registers so that four workgroups share a compute unit.  2: rows of up to REG_ROW_BIG elements at up to 256
// registers (two workgroups per compute unit).  A launch looks only at the rows whose length lies in
// (n_above, n_upto] and leaves the others to the launch of the other variant; rows the single-sweep path turns
// down take the general path on global memory and the plain LDS sorting network.  Rows are taken in ascending
// order (with causal windows the short ones first: 0.118 ms at 8192 x 8192 against 0.161 ms longest first and
// 0.141 ms with short and long rows alternating).
template <bool STAGED, int LEAN>
__global__ __launch_bounds__(BLOCK, LEAN == 1 ? 4 : LEAN == 2 ? 2 : 1) void topk_kernel(
    const float* __restrict__ logits, long ld, const int* __restrict__ row_begin, const int* __restrict__ row_end,
    int width, const int* __restrict__ id_base, int K, int Kp2, int sorted, float* __restrict__ scores,
    int* __restrict__ ids, int nmax, int n_above, int n_upto) {
  extern __shared__ __attribute__((aligned(16))) unsigned char smem[];
  int* hist = (int*)smem;                          // HBINS
  int* scratch = hist + HBINS;                     // 16
  float* outv = (float*)(scratch + 16);            // Kp2
  int* outi = (int*)(outv + Kp2);                  // Kp2
  unsigned* keys = (unsigned*)(outi + Kp2 + 2 * LIN_SPARE);   // nmax (STAGED only); the gap extends the (score, id) buffer
  const int tid = threadIdx.x;
  const long row = blockIdx.x;
  const int cb = max(row_begin ? row_begin[row] : 0, 0);
  const int ce = min(row_end ? row_end[row] : width, width);
  const int n = max(ce - cb, 0);
  if (n <= n_above || n > n_upto) return;
  const int base_id = (id_base ? id_base[row] : 0) + cb;
  const float* src = logits + row * ld + cb;
  float* sv = scores + row * (long)K;
  int* si = ids + row * (long)K;
  (void)nmax;

  auto key_at = [&](int e) -> unsigned { return STAGED ? keys[e] : f2key(src[e]); };

  if (sorted && n > 0) {   // single-sweep path, also for rows shorter than K
    if (STAGED) {
      if (linear_select_sort(src, keys, n, K, base_id, hist, scratch, (unsigned long long*)outv, sv, si)) return;
      __syncthreads();
    } else if (LEAN == 1 && n + 3 <= REG_ROW) {
      bool done;
      unsigned long long* obuf = (unsigned long long*)outv;
      if (n + 3 <= 8 * BLOCK) done = linear_select_sort_regs<2>(src, n, K, base_id, hist, scratch, obuf, sv, si);
      else if (n + 3 <= 16 * BLOCK) done = linear_select_sort_regs<4>(src, n, K, base_id, hist, scratch, obuf, sv, si);
      else done = linear_select_sort_regs<REG_ROW / (4 * BLOCK)>(src, n, K, base_id, hist, scratch, obuf, sv, si);
      if (done) return;
      __syncthreads();
    } else if (LEAN == 2 && n + 3 <= REG_ROW_BIG) {
      bool done;
      unsigned long long* obuf = (unsigned long long*)outv;
      if (n + 3 <= 16 * 4 * BLOCK) done = linear_select_sort_regs<16>(src, n, K, base_id, hist, scratch, obuf, sv, si);
      else if (n + 3 <= 24 * 4 * BLOCK) done = linear_select_sort_regs<24>(src, n, K, base_id, hist, scratch, obuf, sv, si);
      else done = linear_select_sort_regs<REG_ROW_BIG / (4 * BLOCK)>(src, n, K, base_id, hist, scratch, obuf, sv, si);
      if (done) return;
      __syncthreads();
    }
  }
  if (n <= K) {
    for (int t = tid; t < Kp2; t += BLOCK) {
      float v = t < n ? src[t] : -INFINITY;
      outv[t] = v;
      outi[t] = (t < n && v != -INFINITY) ? base_id + t : -1;
    }
  } else {
    if (STAGED && !sorted) {
      for (int e = tid; e < n; e += BLOCK) keys[e] = f2key(src[e]);
    }
    // ---- pass 1: bits [31:20] ------------------------------------------------------------
    for (int b = tid; b < HBINS; b += BLOCK) hist[b] = 0;
    __syncthreads();
    for (int e = tid; e < n; e += BLOCK) atomicAdd(&hist[key_at(e) >> 20], 1);
    __syncthreads();
    Pick p1 = pick_bin(hist, 4096, K, scratch, scratch + 8);
    int need = K - p1.above;
    // ---- pass 2: bits [19:10] among keys in bin p1 -----------------------------------------
    for (int b = tid; b < 1024; b += BLOCK) hist[b] = 0;
    __syncthreads();
    for (int e = tid; e < n; e += BLOCK) {
      unsigned k = key_at(e);
      if ((int)(k >> 20) == p1.bin) atomicAdd(&hist[(k >> 10) & 1023], 1);
    }
    __syncthreads();
    Pick p2 = pick_bin(hist, 1024, need, scratch, scratch + 8);
    need -= p2.above;
    // ---- pass 3: bits [9:0] ----------------------------------------------------------------
    const unsigned pre22 = ((unsigned)p1.bin << 10) | (unsigned)p2.bin;
    for (int b = tid; b < 1024; b += BLOCK) hist[b] = 0;
    __syncthreads();
    for (int e = tid; e < n; e += BLOCK) {
      unsigned k = key_at(e);
      if ((k >> 10) == pre22) atomicAdd(&hist[k & 1023], 1);
    }
    __syncthreads();
    Pick p3 = pick_bin(hist, 1024, need, scratch, scratch + 8);
    const unsigned thr = (pre22 << 10) | (unsigned)p3.bin;   // the K-th largest key
    const int ties = need - p3.above;                         // how many keys == thr to keep (>= 1)
    // ---- compaction in ascending column order ------------------------------------------------
    const int cs = (n + BLOCK - 1) / BLOCK;
    const int e0 = min(tid * cs, n), e1 = min(e0 + cs, n);
    int ngt = 0, neq = 0;
    for (int e = e0; e < e1; e++) { unsigned k = key_at(e); ngt += k > thr; neq += k == thr; }
    int tot;
    const int eq_before = block_exscan(neq, scratch, tot);
    const int eq_take = max(0, min(neq, ties - eq_before));
    int pos = block_exscan(ngt + eq_take, scratch, tot);
    int eq_seen = 0;
    for (int e = e0; e < e1; e++) {
      unsigned k = key_at(e);
      bool take = k > thr;
      if (k == thr) { take = eq_seen < eq_take; eq_seen++; }
      if (take) {
        float v = key2f(k);
        outv[pos] = v;
        outi[pos] = v != -INFINITY ? base_id + e : -1;
        pos++;
      }
    }
    for (int t = K + tid; t < Kp2; t += BLOCK) { outv[t] = -INFINITY; outi[t] = -1; }
  }
  __syncthreads();

  if (sorted) {   // bitonic sort, descending score, ascending id among equal scores
    const int ept = LEAN != 0 ? 0 : Kp2 / BLOCK;
    if (ept == 8) { bitonic_regs<8>(outv, outi, (unsigned long long*)outv, Kp2, sv, si, K); return; }
    else if (ept == 4) { bitonic_regs<4>(outv, outi, (unsigned long long*)outv, Kp2, sv, si, K); return; }
    else if (ept == 2) { bitonic_regs<2>(outv, outi, (unsigned long long*)outv, Kp2, sv, si, K); return; }
    else if (ept == 1) { bitonic_regs<1>(outv, outi, (unsigned long long*)outv, Kp2, sv, si, K); return; }
    else if (ept == 16) { bitonic_regs<16>(outv, outi, (unsigned long long*)outv, Kp2, sv, si, K); return; }
    else if (ept == 32) { bitonic_regs<32>(outv, outi, (unsigned long long*)outv, Kp2, sv, si, K); return; }
    else {
      for (int size = 2; size <= Kp2; size <<= 1) {
        for (int stride = size >> 1; stride > 0; stride >>= 1) {
          for (int t = tid; t < (Kp2 >> 1); t += BLOCK) {
            const int lo = 2 * t - (t & (stride - 1));
            const int hi = lo + stride;
            const bool desc = ((lo & size) == 0);
            const float a = outv[lo], b = outv[hi];
            const int ia = outi[lo], ib = outi[hi];
            if (comes_first(a, ia, b, ib) != desc) { outv[lo] = b; outv[hi] = a; outi[lo] = ib; outi[hi] = ia; }
          }
          __syncthreads();
        }
      }
    }
  }
  for (int t = tid; t < K; t += BLOCK) { sv[t] = outv[t]; si[t] = outi[t]; }
}

}  // namespace

int dsa_topk_launch(const float* logits, int S, int64_t ld, const int32_t* row_begin, const int32_t* row_end,
                    int width, const int32_t* id_base, int K, int sorted, float* scores, int32_t* ids,
                    hipStream_t st) {
  DSA_REQUIRE(S >= 0 && width > 0 && ld >= width && K > 0, "dsa_topk: bad sizes S=%d width=%d K=%d", S, width, K);
  DSA_REQUIRE(K <= 8192, "dsa_topk: K=%d exceeds the supported maximum 8192", K);
  if (S == 0) return DSA_OK;
  int Kp2 = 1;
  while (Kp2 < K) Kp2 <<= 1;
  const size_t fixed = (size_t)HBINS * 4 + 64 + (size_t)Kp2 * 8 + (size_t)LIN_SPARE * 8;
  const size_t staged = fixed + (size_t)width * 4;
  // sorted rows that fit a register variant need no staging buffer: rows of up to REG_ROW elements go to the
  // 128-register kernel (four workgroups per compute unit), longer ones up to REG_ROW_BIG to its 256-register
  // form in a second launch; each launch skips the other's rows
  const bool lean = sorted && width + 3 <= REG_ROW_BIG;
  const bool use_staged = !lean && staged <= 160 * 1024;
  const size_t smem = use_staged ? staged : fixed;
  const int none = 0x7fffffff;
  if (lean) {
    auto k1 = topk_kernel<false, 1>;
    auto k2 = topk_kernel<false, 2>;
    if (dsa_reserve_lds((const void*)k1, smem) != hipSuccess ||
        dsa_reserve_lds((const void*)k2, smem) != hipSuccess)
      DSA_FAIL(DSA_ERR_LAUNCH, "dsa_topk: cannot reserve %zu bytes of LDS", smem);
    const int split = REG_ROW - 3;
    k1<<<dim3(S), dim3(BLOCK), smem, st>>>(logits, (long)ld, row_begin, row_end, width, id_base, K, Kp2, sorted, scores, ids,
                                           width, -1, split);
    if (width > split)
      k2<<<dim3(S), dim3(BLOCK), smem, st>>>(logits, (long)ld, row_begin, row_end, width, id_base, K, Kp2, sorted, scores,
                                             ids, width, split, none);
  } else {
    auto kern = use_staged ? topk_kernel<true, 0> : topk_kernel<false, 0>;
    if (dsa_reserve_lds((const void*)kern, smem) != hipSuccess)
      DSA_FAIL(DSA_ERR_LAUNCH, "dsa_topk: cannot reserve %zu bytes of LDS", smem);
    kern<<<dim3(S), dim3(BLOCK), smem, st>>>(logits, (long)ld, row_begin, row_end, width, id_base, K, Kp2, sorted, scores, ids,
                                             width, -1, none);
  }
  DSA_CHECK_LAUNCH("dsa_topk");
  return DSA_OK;
}

extern "C" int dsa_topk(const float* logits, int S, int64_t ld, const int32_t* row_begin, const int32_t* row_end,
                        int width, const int32_t* id_base, int K, int sorted, float* scores, int32_t* ids,
                        void* stream) {
  return dsa_topk_launch(logits, S, ld, row_begin, row_end, width, id_base, K, sorted, scores, ids,
                         (hipStream_t)stream);
}

// ---- fused indexer forward: logits of one query block at a time, then its top-k ----------------
int dsa_indexer_logits_block(const void* q8, const float* q_w, const void* k8, const float* k_scale,
                             const int32_t* ks, const int32_t* ke, int S, int Hi, int Sk, float* logits,
                             int64_t ld, int width, int relative, int clean, int q_begin, int q_count,
                             hipStream_t st);

static int fused_block_rows(int Sk) {
  // one block's logits stay within the 256 MiB memory-side cache where that still leaves a block 8192 queries:
  // 1024 workgroups of 8 queries, four rounds over the 256 compute units (blocks of 2048 queries - one workgroup per
  // compute unit, half of what fits - took 2.6 ms for 32768 packed tokens where blocks of 8192 take 1.9 ms)
  long rows = (256l << 20) / ((long)Sk * 4);
  rows = rows < 8192 ? 8192 : rows;
  return (int)(rows / 8 * 8);
}

extern "C" size_t dsa_indexer_topk_workspace_bytes(int S, int Sk, int K) {
  (void)K;
  int rows = fused_block_rows(Sk);
  if (rows > S) rows = (S + 7) / 8 * 8;
  return (size_t)rows * (size_t)Sk * 4;
}

// Logits of `rows` queries at a time into lg ([rows][Sk] floats), then their top-k.
static int indexer_topk_blocks(const void* q8, const float* q_w, const void* k8, const float* k_scale, const int32_t* ks,
                               const int32_t* ke, int S, int Hi, int Sk, int K, int sorted, float* scores, int32_t* ids,
                               float* lg, int rows, hipStream_t st) {
  for (int q0 = 0; q0 < S; q0 += rows) {
    const int cnt = S - q0 < rows ? S - q0 : rows;
    int rc = dsa_indexer_logits_block(q8, q_w, k8, k_scale, ks, ke, S, Hi, Sk, lg, Sk, Sk, 0, 0, q0, cnt, st);
    if (rc != DSA_OK) return rc;
    rc = dsa_topk_launch(lg, cnt, Sk, ks + q0, ke + q0, Sk, nullptr, K, sorted, scores + (size_t)q0 * K,
                         ids + (size_t)q0 * K, st);
    if (rc != DSA_OK) return rc;
  }
  return DSA_OK;
}

extern "C" int dsa_indexer_topk_fwd(const void* q8, const float* q_w, const void* k8, const float* k_scale,
                                    const int32_t* ks, const int32_t* ke, int S, int Hi, int Sk, int K, int sorted,
                                    float* scores, int32_t* ids, void* workspace, size_t workspace_bytes,
                                    void* stream) {
  if (S == 0) return DSA_OK;
  DSA_REQUIRE(workspace != nullptr && workspace_bytes >= dsa_indexer_topk_workspace_bytes(S, Sk, K),
              "dsa_indexer_topk_fwd: workspace of %zu bytes is too small", workspace_bytes);
  return indexer_topk_blocks(q8, q_w, k8, k_scale, ks, ke, S, Hi, Sk, K, sorted, scores, ids, (float*)workspace,
                             fused_block_rows(Sk), (hipStream_t)stream);
}

// ---- the same without any allocation by anyone: the logits blocks live in a device array of the library ----
// For callers that cannot allocate device memory (code under HIP graph capture, tight serving loops):
// they pass inputs and outputs only.  Every GPU the library runs on holds its own copy of the array
// until the process ends; calls that overlap on one GPU share it and race - order them on one stream.
constexpr size_t STATIC_SCRATCH_BYTES = (size_t)64 << 20;
constexpr int STATIC_MIN_ROWS = 256;           // a block of fewer queries would leave most compute units idle
static __device__ __align__(256) unsigned char scratch[STATIC_SCRATCH_BYTES];

#include <mutex>
static std::mutex scratch_mutex;
static void* scratch_ptr[64];                  // per device: the array's address on that device (0 = not asked yet)

extern "C" int dsa_indexer_topk_fwd_static(const void* q8, const float* q_w, const void* k8, const float* k_scale,
                                           const int32_t* ks, const int32_t* ke, int S, int Hi, int Sk, int K,
                                           int sorted, float* scores, int32_t* ids, void* stream) {
  if (S == 0) return DSA_OK;
  DSA_REQUIRE(Sk > 0 && (size_t)Sk * 4 * STATIC_MIN_ROWS <= STATIC_SCRATCH_BYTES,
              "dsa_indexer_topk_fwd_static: at most %zu keys fit the library's %zu MiB scratch array, got %d "
              "(use dsa_indexer_topk_fwd with a workspace)",
              STATIC_SCRATCH_BYTES / (4 * STATIC_MIN_ROWS), STATIC_SCRATCH_BYTES >> 20, Sk);
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64)
    DSA_FAIL(DSA_ERR_LAUNCH, "dsa_indexer_topk_fwd_static: no current device");
  void* base;
  {
    std::lock_guard<std::mutex> lock(scratch_mutex);
    if (scratch_ptr[dev] == nullptr) {         // first call on this device: the array's address here
      void* p = nullptr;
      const hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(scratch));
      if (e != hipSuccess || p == nullptr)
        DSA_FAIL(DSA_ERR_LAUNCH, "dsa_indexer_topk_fwd_static: hipGetSymbolAddress failed: %s", hipGetErrorString(e));
      scratch_ptr[dev] = p;
    }
    base = scratch_ptr[dev];
  }
  int rows = (int)(STATIC_SCRATCH_BYTES / ((size_t)Sk * 4)) / 8 * 8;
  // (nothing in the array has to start at zero: the logits kernel writes columns [ks, ke) of every row of a block
  // and the selection reads no others)
  return indexer_topk_blocks(q8, q_w, k8, k_scale, ks, ke, S, Hi, Sk, K, sorted, scores, ids, (float*)base, rows,
                             (hipStream_t)stream);
}
