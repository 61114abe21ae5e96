// Lightning-indexer logits for gfx950: fp8-e4m3 MFMA GEMM with the ReLU, the head-weight
// reduction and the per-key scale fused into the epilogue.
//
//   logits[i, j] = k_scale[j] * sum_h q_w[i,h] * relu(q8[i,h,:] . k8[j,:])      ks[i] <= j < ke[i]
//
// One workgroup owns 8 consecutive queries, one per wave (512 threads; at 122 registers per lane
// four waves share a SIMD), and streams the keys its queries can see through LDS in tiles of 128
// rows (global_load_lds, double buffered, 16-byte slots XOR-swizzled per row).  For every 32-key
// sub-tile a wave issues, per group of 32 heads, two v_mfma_f32_32x32x64_f8f6f4 (A = the query's fp8
// rows, held in registers for the whole sweep; B = key rows from LDS).  The accumulator layout puts
// one key per lane and 16 heads per register file column, so the weighted ReLU-sum over heads is 2
// VALU ops per element inside a lane plus one exchange between the two half-waves.  Per sub-tile
// that is 4 MFMAs of 64 cycles against about 77 VALU issues of 4 cycles: the VALU port is the busier
// of the two, and the matrix pipe of one wave overlaps the epilogue of the others, not its own -
// hence the small register footprint and the high occupancy.  HBM is far from binding (q8 / k8 are
// read once, logits written once).
#include "dsa_common.h"

namespace {

constexpr int D = 128;          // indexer head dim (bytes per fp8 row)
constexpr int BK = 128;         // keys per LDS tile
constexpr int TILE_BYTES = BK * D;
constexpr int QB = 8;           // queries per workgroup

__device__ __forceinline__ int swz(int r) { return (r & 7) ^ ((r >> 3) & 1); }

__device__ __forceinline__ void dma16(unsigned lds_base, unsigned goff, const void* gbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %1, %2"
               :: "s"(lds_base), "v"(goff), "s"(gbase) : "memory");
}
__device__ __forceinline__ void dma4(unsigned lds_base, unsigned goff, const void* gbase) {
  asm volatile("s_mov_b32 m0, %0\n\ts_nop 0\n\tglobal_load_lds_dword %1, %2"
               :: "s"(lds_base), "v"(goff), "s"(gbase) : "memory");
}

// max(x, 0) as one instruction, on the bit pattern (a negative float is a negative integer):
// fmaxf would first quiet a possible signalling NaN with a second v_max, which doubles the cost
// of the epilogue.
__device__ __forceinline__ float relu1(float x) {
  return __builtin_bit_cast(float, max(__builtin_bit_cast(int, x), 0));
}

__global__ void fill_neg_inf_kernel(float* __restrict__ p, long rows, long ld, int width) {
  const long n = rows * (long)width;
  for (long e = (long)blockIdx.x * blockDim.x + threadIdx.x; e < n; e += (long)gridDim.x * blockDim.x)
    p[(e / width) * ld + (e % width)] = -INFINITY;
}

// sum of x over the two half-waves (lanes l and l ^ 32), in every lane.  v_permlane32_swap
// exchanges the upper half of its first operand with the lower half of its second: afterwards one
// register holds the lower-half values in both halves and the other the upper-half values.  (Written
// as inline assembly: given the same value for both operands the compiler's builtin is folded as if
// both results were equal.)
__device__ __forceinline__ float add_halves(float x) {
  float a = x, b = x;
  asm volatile("s_nop 1\n\tv_permlane32_swap_b32 %0, %1\n\ts_nop 1" : "+v"(a), "+v"(b));
  return a + b;
}

template <int NHT>   // groups of 32 heads
__global__ __launch_bounds__(64 * QB, 4) void indexer_logits_kernel(
    const unsigned char* __restrict__ q8, const float* __restrict__ q_w, const unsigned char* __restrict__ k8,
    const float* __restrict__ k_scale, const int* __restrict__ ks, const int* __restrict__ ke,
    int S, int Sk, float* __restrict__ logits, long ld, int relative, int q_begin, int q_count) {
  __shared__ __attribute__((aligned(1024))) unsigned char smem[2 * TILE_BYTES + 2 * BK * 4];
  constexpr int HI = NHT * 32;
  constexpr int NWAVE = QB;
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // scalar: window tests below become scalar branches
  const int r = lane & 31, g = lane >> 5;
  const int nblk = (q_count + QB - 1) / QB;
  const int blk = nblk - 1 - (int)blockIdx.x;            // longest windows first
  const int qb0 = q_begin + blk * QB;
  const int q_end = q_begin + q_count;

  // window union of the block
  int jlo = 0x7fffffff, jhi = 0;
  for (int t = 0; t < QB; t++) {
    const int i = qb0 + t;
    if (i < q_end) { jlo = min(jlo, ks[i]); jhi = max(jhi, min(ke[i], Sk)); }
  }
  jlo = max(jlo, 0);

  // this wave's query
  const int i_q = qb0 + wave;
  const bool live = i_q < q_end;
  const int qi = live ? i_q : -1;
  const int qks = live ? max(ks[i_q], 0) : 0;
  const int qke = live ? min(ke[i_q], Sk) : 0;
  const int wlo = live ? qks : 0x7fffffff, whi = live ? qke : 0;     // the wave's window
  i32x8 aq[NHT][2];
  float wq[NHT][16];
  {
    const int is = live ? i_q : qb0;
#pragma unroll
    for (int t = 0; t < NHT; t++) {
      const unsigned char* row = q8 + ((size_t)is * HI + 32 * t + r) * D + 32 * g;
#pragma unroll
      for (int s = 0; s < 2; s++) {
        const i32x4 lo = *(const i32x4*)(row + 64 * s);
        const i32x4 hi = *(const i32x4*)(row + 64 * s + 16);
        aq[t][s] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      }
      const float* wrow = q_w + (size_t)is * HI + 32 * t + 4 * g;
#pragma unroll
      for (int j = 0; j < 4; j++) {
        const f32x4 w4 = *(const f32x4*)(wrow + 8 * j);
#pragma unroll
        for (int e = 0; e < 4; e++) wq[t][4 * j + e] = w4[e];
      }
    }
  }
  DSA_WAIT_VMCNT(0);
#pragma unroll
  for (int t = 0; t < NHT; t++)
#pragma unroll
    for (int s = 0; s < 2; s++) asm volatile("" : "+v"(aq[t][s]));

  const int t_lo = jlo / BK, t_hi = (jhi + BK - 1) / BK;      // key tiles [t_lo, t_hi)
  const unsigned lds0 = (unsigned)(uintptr_t)smem;
  const int gkey = tid >> 3, gsub = tid & 7;                  // 8 NWAVE key rows per DMA instruction
  auto issue = [&](int t) {
    const unsigned lb = lds0 + (unsigned)((t & 1) * TILE_BYTES + wave * 1024);
#pragma unroll
    for (int c = 0; c < BK / (8 * NWAVE); c++) {
      const int key = c * 8 * NWAVE + gkey;
      const int row = min(t * BK + key, Sk - 1);
      dma16(lb + c * 1024 * NWAVE, (unsigned)row * D + (unsigned)((gsub ^ swz(key)) * 16), k8);
    }
    if (wave < BK / 64) {   // the tile's per-key scales
      const unsigned sb = lds0 + (unsigned)(2 * TILE_BYTES + (t & 1) * BK * 4 + wave * 256);
      dma4(sb, (unsigned)min(t * BK + wave * 64 + lane, Sk - 1) * 4u, k_scale);
    }
  };
  // B operand of sub-tile c: key row 32c + r, bytes [64s + 32g, +32) = 16-byte slots 4s+2g, 4s+2g+1
  unsigned b_off[2][2];
#pragma unroll
  for (int s = 0; s < 2; s++)
#pragma unroll
    for (int x = 0; x < 2; x++) b_off[s][x] = (unsigned)(r * D + (((4 * s + 2 * g + x) ^ swz(r)) << 4));

  if (t_lo < t_hi) issue(t_lo);
  for (int t = t_lo; t < t_hi; t++) {
    DSA_WAIT_VMCNT(0);
    __syncthreads();
    if (t + 1 < t_hi) issue(t + 1);
    const unsigned char* tb = smem + (t & 1) * TILE_BYTES;
    const float* ksc_s = (const float*)(smem + 2 * TILE_BYTES) + (t & 1) * BK;
#pragma unroll 1
    for (int c = 0; c < BK / 32; c++) {
      const int j0 = t * BK + c * 32;
      if (j0 >= whi || j0 + 32 <= wlo) continue;               // scalar: nothing of this wave's windows here
      const int j = j0 + r;
      const unsigned char* cb = tb + c * 32 * D;
      i32x8 bk[2];
#pragma unroll
      for (int s = 0; s < 2; s++) {
        const i32x4 lo = *(const i32x4*)(cb + b_off[s][0]);
        const i32x4 hi = *(const i32x4*)(cb + b_off[s][1]);
        bk[s] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
      }
      const float ksc = ksc_s[c * 32 + r];
      float part = 0.f;
#pragma unroll
      for (int tt = 0; tt < NHT; tt++) {
        f32x16 acc;
#pragma unroll
        for (int e = 0; e < 16; e++) acc[e] = 0.f;
        acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(aq[tt][0], bk[0], acc, 0, 0, 0, 127, 0, 127);
        acc = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(aq[tt][1], bk[1], acc, 0, 0, 0, 127, 0, 127);
#pragma unroll
        for (int e = 0; e < 16; e++) part = fmaf(wq[tt][e], relu1(acc[e]), part);
      }
      part = add_halves(part) * ksc;
      if (g == 0 && j >= qks && j < qke) {
        const int col = relative ? j - qks : j;
        logits[(size_t)(qi - q_begin) * ld + col] = part;
      }
    }
  }
}

}  // namespace

// q_begin/q_count select a block of queries; row 0 of `logits` is query q_begin.
int dsa_indexer_logits_block(const void* q8, const float* q_w, const void* k8, const float* k_scale,
                             const int32_t* ks, const int32_t* ke, int S, int Hi, int Sk, float* logits,
                             int64_t ld, int width, int relative, int clean, int q_begin, int q_count,
                             hipStream_t st) {
  DSA_REQUIRE(Hi == 32 || Hi == 64, "dsa_indexer_logits: head count must be 32 or 64, got %d", Hi);
  DSA_REQUIRE(S >= 0 && Sk > 0 && width > 0 && ld >= width, "dsa_indexer_logits: bad sizes S=%d Sk=%d width=%d", S, Sk, width);
  DSA_REQUIRE((size_t)Sk * D <= 0xffffffffull, "dsa_indexer_logits: key array too large");
  DSA_REQUIRE(((uintptr_t)q8 % 16) == 0 && ((uintptr_t)k8 % 16) == 0 && ((uintptr_t)q_w % 16) == 0,
              "dsa_indexer_logits: misaligned pointer");
  DSA_REQUIRE(q_begin >= 0 && q_begin + q_count <= S, "dsa_indexer_logits: bad query block");
  if (q_count <= 0) return DSA_OK;
  if (clean) {
    fill_neg_inf_kernel<<<dim3(2048), dim3(256), 0, st>>>(logits, q_count, (long)ld, width);
    DSA_CHECK_LAUNCH("dsa_indexer_logits(fill)");
  }
  dim3 grid((q_count + QB - 1) / QB), block(64 * QB);
#define DSA_IDX_LAUNCH(N) indexer_logits_kernel<N><<<grid, block, 0, st>>>( \
    (const unsigned char*)q8, q_w, (const unsigned char*)k8, k_scale, ks, ke, S, Sk, logits, (long)ld, relative, q_begin, q_count)
  if (Hi == 32) DSA_IDX_LAUNCH(1);
  else DSA_IDX_LAUNCH(2);
#undef DSA_IDX_LAUNCH
  DSA_CHECK_LAUNCH("dsa_indexer_logits");
  return DSA_OK;
}

extern "C" int dsa_indexer_logits(const void* q8, const float* q_w, const void* k8, const float* k_scale,
                                  const int32_t* ks, const int32_t* ke, int S, int Hi, int Sk, float* logits,
                                  int64_t ld, int width, int relative, void* stream) {
  return dsa_indexer_logits_block(q8, q_w, k8, k_scale, ks, ke, S, Hi, Sk, logits, ld, width, relative, 1, 0, S,
                                  (hipStream_t)stream);
}
